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


def test_rollback_gives_back_what_no_commit_filled():
    c = CacheManager([(0, True, FULL, None), (1, True, WIN, None)], 8, {FULL: 12, WIN: 8}, 2)
    c.add_request("r")
    c.reserve("r", 13)
    c.commit("r", 13)
    held = [list(c.block_table(g, "r")) for g in range(2)]
    used = [g.pool.num_used for g in c.groups]
    c.reserve("r", 30)                       # a step that then fails
    assert c.groups[0].pool.num_used == 6
    assert c.rollback("r") == 2 * 4
    assert [list(c.block_table(g, "r")) for g in range(2)] == held
    assert [g.pool.num_used for g in c.groups] == used and c.num_tokens("r") == 13
    assert c.rollback("r") == 0              # nothing left to give back
    c.check()
    c.reserve("r", 3)                        # fits the page it has: nothing taken, nothing to roll back
    assert c.rollback("r") == 0
    c.commit("r", 3)
    c.release("r")
    c.check()


def test_padding_slot_is_no_requests_slot():
    c = CacheManager([(0, True, FULL, None), (1, True, None, StateSpec((4,)))], 8, 4, 3)
    slots = [c.add_request(i) for i in range(3)]
    assert c.padding_slot not in slots and sorted(slots) == [0, 1, 2]
    import torch
    c2 = CacheManager([(0, True, FULL, None), (1, True, None, StateSpec((4,)))], 8, 4, 3, dtype=torch.float32,
                      device="cpu")
    assert c2.state_tensors[1].shape == (4, 4)      # a row more than there are requests


def test_window_pool_never_runs_short():
    """A group with a window, sized by window_pool_pages, serves any schedule of portions that
    keeps to the token budget, however long the requests grow."""
    from tffinfer_amd.cache.sizing import window_pool_pages
    rng = random.Random(5)
    ps, window, seqs, budget = 8, 24, 4, 64
    n = window_pool_pages(window, ps, seqs, budget)
    c = CacheManager([(0, True, WIN, None)], ps, n, seqs)
    for r in range(seqs):
        c.add_request(r)
    for _ in range(300):
        left = budget
        portions = {}
        for r in range(seqs):
            k = rng.choice([0, 1, 1, 2, 7, 30, 64])
            k = min(k, left)
            if k:
                portions[r] = k
                left -= k
        for r, k in portions.items():
            c.reserve(r, k)                  # never raises OutOfPages
        for r, k in portions.items():
            c.commit(r, k)
        c.check()
    assert max(c.num_tokens(r) for r in range(seqs)) > 50 * ps


def test_plan_pages_sizes_groups_by_their_need():
    from tffinfer_amd.cache.sizing import bytes_per_page, plan_pages, state_bytes, window_pool_pages
    import torch
    reqs = [(0, True, FULL, None), (1, True, WIN, None), (2, True, WIN, None), (3, True, None, StateSpec((100,), torch.float32))]
    ps, seqs, budget = 8, 4, 64
    pages = plan_pages(reqs, ps, 2, seqs, budget, tokens=4000)
    assert pages[FULL] == 500 + seqs
    assert pages[WIN] == window_pool_pages(24, ps, seqs, budget) < 40
    # bytes: the window groups first, the rest to the group that keeps every key
    per_full, per_win = bytes_per_page(FULL, 1, ps, 2), bytes_per_page(WIN, 2, ps, 2)
    kv = 100 * per_full + pages[WIN] * per_win + 5
    by = plan_pages(reqs, ps, 2, seqs, budget, kv_bytes=kv)
    assert by[WIN] == pages[WIN] and by[FULL] == 100
    # the free memory caps what the tokens ask for, and the state tensors come off it first
    assert state_bytes(reqs, seqs) == 5 * 100 * 4
    capped = plan_pages(reqs, ps, 2, seqs, budget, tokens=4000, free_bytes=kv + state_bytes(reqs, seqs))
    assert capped[FULL] == 100 and capped[WIN] == pages[WIN]
    # a request's short cache never asks a window group for more than the group that keeps all
    small = plan_pages(reqs, ps, 2, seqs, budget, tokens=40)
    assert small[FULL] == 5 + seqs and small[WIN] == small[FULL]
    with pytest.raises(ValueError, match="holds no page"):
        plan_pages(reqs, ps, 2, seqs, budget, kv_bytes=10)
    assert plan_pages([(0, True, None, None)], ps, 2, seqs, budget, tokens=10) == {}
