"""The cache manager on the host: no page lost, held twice or freed twice,
under random orders of requests; windows give pages back; slots."""
import random

import pytest

from tffinfer_amd.cache import BlockPool, CacheManager, OutOfPages, OutOfSlots, StateSlots
from tffinfer_amd.parts.base import KVCacheSpec, StateSpec

FULL = KVCacheSpec(2, 16, 0)
WIN = KVCacheSpec(2, 16, 24)


def test_pool_all_or_nothing_and_reuse():
    p = BlockPool(4)
    a = p.allocate(3)
    assert a == [0, 1, 2] and p.num_free == 1
    with pytest.raises(OutOfPages):
        p.allocate(2)
    assert p.num_free == 1          # nothing was taken
    p.free([1])
    assert p.allocate(1) == [1]     # the page just freed comes back first
    with pytest.raises(ValueError, match="twice"):
        p.free([0, 0])
    p.check()


def test_pool_rejects_foreign_page():
    p = BlockPool(2)
    with pytest.raises(ValueError):
        p.free([5])
    with pytest.raises(ValueError, match="twice"):
        p.free([1])     # never allocated


def test_slots():
    s = StateSlots(2)
    a, b = s.acquire(), s.acquire()
    assert {a, b} == {0, 1}
    with pytest.raises(OutOfSlots):
        s.acquire()
    s.release(a)
    with pytest.raises(ValueError):
        s.release(a)
    assert s.acquire() == a
    s.check()


def mk(num_pages=16, ps=8, max_seqs=4, specs=(FULL, FULL, WIN)):
    reqs = [(i, True, s, None) for i, s in enumerate(specs)]
    return CacheManager(reqs, ps, num_pages, max_seqs)


def test_groups_by_need():
    c = mk()
    assert len(c.groups) == 2
    assert c.groups[0].cache_ids == [0, 1] and c.groups[1].cache_ids == [2]
    assert c.group_index(2) == 1


def test_growth_and_slot_mapping():
    c = mk(specs=(FULL,))
    c.add_request("r")
    assert c.pages_needed("r", 9) == [2]
    c.reserve("r", 9)
    assert c.slot_mapping(0, "r", 0, 9) == [0, 1, 2, 3, 4, 5, 6, 7, 8]
    c.commit("r", 9)
    assert c.pages_needed("r", 7) == [0] and c.pages_needed("r", 8) == [1]
    c.add_request("q")
    c.reserve("q", 3)
    assert c.slot_mapping(0, "q", 0, 3) == [16, 17, 18]
    c.commit("q", 3)
    c.reserve("r", 8)
    assert c.slot_mapping(0, "r", 9, 8)[-1] == 3 * 8 + 0     # r's third page is pool page 3
    c.commit("r", 8)
    c.release("r")
    c.add_request("s")
    c.reserve("s", 1)
    assert c.block_table(0, "s") == [3]      # the page freed last is used again first
    c.check()


def test_reserve_is_all_or_nothing_across_groups():
    c = CacheManager([(0, True, FULL, None), (1, True, WIN, None)], 8, {FULL: 4, WIN: 1}, 2)
    c.add_request("r")
    with pytest.raises(OutOfPages):
        c.reserve("r", 9)        # the window group has one page only
    assert c.groups[0].pool.num_free == 4 and c.block_table(0, "r") == []
    c.check()


def test_window_gives_pages_back():
    c = CacheManager([(0, True, FULL, None), (1, True, WIN, None)], 8, {FULL: 12, WIN: 8}, 2)
    c.add_request("r")
    n = 0
    for step in [20, 1, 1, 10, 1, 30, 1, 1]:
        c.reserve("r", step)
        c.commit("r", step)
        n += step
        full, win = c.block_table(0, "r"), c.block_table(1, "r")
        assert all(p >= 0 for p in full) and len(full) == -(-n // 8)
        # every key a later query can reach is still there: positions >= n - 24 + 1
        first_needed = max(0, n - 24 + 1) // 8
        assert all(p >= 0 for p in win[first_needed:])
        assert all(p < 0 for p in win[:max(0, (n - 24 + 1) // 8)])
        assert c.groups[1].pool.num_used <= 24 // 8 + 2
        c.check()
    with pytest.raises(RuntimeError, match="given back"):
        c.slot_mapping(1, "r", 0, 1)
    c.release("r")
    assert c.groups[0].pool.num_used == 0 and c.groups[1].pool.num_used == 0


def test_request_twice_and_unknown():
    c = mk()
    c.add_request("r")
    with pytest.raises(ValueError, match="already"):
        c.add_request("r")
    with pytest.raises(KeyError):
        c.release("nobody")


def test_read_without_writer_is_refused():
    with pytest.raises(ValueError, match="no layer call writes"):
        CacheManager([(0, False, FULL, None)], 8, 4, 2)
    with pytest.raises(ValueError, match="different caches"):
        CacheManager([(0, True, FULL, None), (0, False, WIN, None)], 8, 4, 2)
    c = CacheManager([(0, True, FULL, None), (0, False, FULL, None), (1, True, None, StateSpec((4,)))], 8, 4, 2)
    assert len(c.groups) == 1 and c.groups[0].cache_ids == [0]


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    c = mk(num_pages=24, ps=8, max_seqs=5)
    live = {}
    next_id = 0
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            c.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            r = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 13, 40])
            if c.can_reserve(r, n):
                c.reserve(r, n)
                sm = c.slot_mapping(0, r, live[r], n)
                assert len(set(sm)) == n
                c.commit(r, n)
                live[r] += n
            else:
                before = [g.pool.num_free for g in c.groups]
                with pytest.raises(OutOfPages):
                    c.reserve(r, n)
                assert before == [g.pool.num_free for g in c.groups]
        elif live:
            r = rng.choice(list(live))
            c.release(r)
            del live[r]
        c.check()
        for r, n in live.items():
            assert c.num_tokens(r) == n
    for r in list(live):
        c.release(r)
    c.check()
    assert all(g.pool.num_used == 0 for g in c.groups) and c.slots.num_free == 5
