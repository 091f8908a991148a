"""The host tables of a decode graph against the cache manager's own block
tables, through schedules in which a request's pages change owner: preemption
and recomputation under the same id, an id that is freed and used again, rows
that change place between buckets.  Whatever the history, every row that a
step fills must say what ``cache.block_table`` says (a location is a table
lookup, src/core/runtime/KVCache.h:221-240; a kept copy has to agree with it)."""
import random

import numpy as np
import pytest

from tffinfer_amd.cache import CacheManager
from tffinfer_amd.engine.batch import StepEntry
from tffinfer_amd.engine.graphs import DecodeTables, graph_buckets
from tffinfer_amd.engine.scheduler import Request, Scheduler, SchedulerOptions
from tffinfer_amd.parts.base import KVCacheSpec

from test_key_runs import check_runs

FULL = KVCacheSpec(2, 16, 0)
WIN = KVCacheSpec(2, 16, 16)


def check_rows(tables: DecodeTables, cache, entries):
    o, hv, ps = tables.offs, tables.hv, cache.page_size
    for r, e in enumerate(entries):
        P = cache.num_tokens(e.req)
        assert hv[o[0] + r] == e.tokens[0]
        assert hv[o[1] + r] == P and hv[o[4] + r] == P and hv[o[5] + r] == P + 1
        assert hv[o[6] + r] == cache.slot(e.req)
        for gi, g in enumerate(cache.groups):
            true = cache.block_table(gi, e.req)
            row = tables.block_table_row(gi, r)
            first_live = 0 if g.spec.window == 0 else max(0, (P + 1 - g.spec.window) // ps)
            for b in range(first_live, len(true)):
                assert row[b] == true[b], (f"row {r} request {e.req!r} group {gi} block {b}: "
                                           f"graph says {row[b]}, the cache {true[b]}")
            assert hv[o[10 + 4 * gi] + r] == true[P // ps] * ps + P % ps
    for r in range(len(entries), tables.B):       # padding writes no key and reads position 0 only
        assert hv[o[5] + r] == 1 and hv[o[1] + r] == 0
        for gi in range(len(cache.groups)):
            assert hv[o[10 + 4 * gi] + r] == -1
    # the keys of every row, padding included, dealt into runs: each visible key in exactly one
    for gi, g in enumerate(cache.groups):
        cap = tables.run_caps[gi]
        start = hv[o[12 + 4 * gi]:o[12 + 4 * gi] + tables.B + 1]
        check_runs(hv[o[11 + 4 * gi]:o[11 + 4 * gi] + 4 * cap].reshape(-1, 4), start, hv[o[4]:o[4] + tables.B], g.spec.window)
        assert tables.variant[0] or start[tables.B] == tables.B, "rows of several runs, and a variant that merges nothing"


class TableRunner:
    """Stands where the step function stands: decode-only plans go through the
    tables of their bucket (as ModelRunner._step_graph does) and are checked."""

    def __init__(self, cache, max_seqs, max_len):
        self.cache = cache
        self.buckets = graph_buckets(max_seqs)
        self.tables = {}
        self.max_len = max_len
        self.graph_steps = 0
        self.rng = random.Random(7)

    def run(self, plan):
        sampled = {}
        if all(p.count == 1 for p in plan):
            entries = [StepEntry(p.request.id, [p.request.tokens[p.start]], [0]) for p in plan]
            bucket = next(b for b in self.buckets if b >= len(entries))
            t = self.tables.get(bucket)
            if t is None:
                t = self.tables[bucket] = DecodeTables(self.cache, bucket, self.max_len)
            t.fill(entries)
            check_rows(t, self.cache, entries)
            self.graph_steps += 1
        for p in plan:
            self.cache.commit(p.request.id, p.count)
            if p.samples:
                sampled[p.request.id] = self.rng.randrange(1, 50)
        return sampled


def drive(seed, specs, num_pages, ps, max_seqs, n_requests):
    rng = random.Random(seed)
    max_len = 160
    cache = CacheManager([(i, True, s, None) for i, s in enumerate(specs)], ps, num_pages, max_seqs)
    sched = Scheduler(cache, SchedulerOptions(max_seqs, 48, 16), max_len)
    runner = TableRunner(cache, max_seqs, max_len)
    pending = [Request(i, [rng.randrange(1, 50) for _ in range(rng.randrange(1, 40))],
                       max_new_tokens=rng.randrange(4, 60), ignore_eos=True) for i in range(n_requests)]
    steps = 0
    while sched.has_work or pending:
        while pending and rng.random() < 0.3:     # staggered arrivals
            sched.add_request(pending.pop(0))
        if not sched.has_work:
            sched.add_request(pending.pop(0))
        plan = sched.schedule()
        assert plan
        sched.update(plan, runner.run(plan))
        cache.check()
        steps += 1
        assert steps < 5000
    return sched.stats.preemptions, runner.graph_steps


@pytest.mark.parametrize("specs", [(FULL,), (FULL, WIN)], ids=["full", "full+window"])
def test_rows_equal_the_block_tables_through_preemptions(specs):
    preemptions = graph_steps = 0
    for seed in range(60):
        p, g = drive(seed, specs, num_pages=14, ps=8, max_seqs=3, n_requests=7)
        preemptions += p
        graph_steps += g
    assert preemptions > 50 and graph_steps > 1000     # the schedules do preempt and do decode


def test_a_preempted_request_comes_back_to_its_row_with_other_pages():
    """The failing case, by hand: request 1 decodes in row 1, is preempted, request 0 takes a
    page meanwhile, request 1 is added again (same id, pages in another order) and decodes in
    row 1 again."""
    cache = CacheManager([(0, True, FULL, None)], 8, 6, 2)
    t = DecodeTables(cache, 2, 64)
    for rid, n in ((0, 8), (1, 16)):
        cache.add_request(rid)
        cache.reserve(rid, n)
        cache.commit(rid, n)
    ents = [StepEntry(0, [5], [0]), StepEntry(1, [6], [0])]
    for e in ents:
        cache.reserve(e.req, 1)
    t.fill(ents)
    check_rows(t, cache, ents)
    for e in ents:
        cache.commit(e.req, 1)
    before = list(cache.block_table(0, 1))
    cache.release(1)                                   # preempted
    cache.reserve(0, 8)                                # the other one grows into a freed page
    cache.commit(0, 7)
    cache.add_request(1)                               # and comes back
    cache.reserve(1, 17)
    cache.commit(1, 17)
    assert cache.block_table(0, 1) != before and len(cache.block_table(0, 1)) == len(before)
    for e in ents:
        cache.reserve(e.req, 1)
    t.fill(ents)
    check_rows(t, cache, ents)


def test_an_id_freed_and_used_again():
    cache = CacheManager([(0, True, FULL, None)], 8, 8, 2)
    t = DecodeTables(cache, 1, 64)
    cache.add_request("a")
    cache.add_request("b")
    cache.reserve("b", 3)
    cache.reserve("a", 20)
    cache.commit("a", 20)
    e = [StepEntry("a", [1], [0])]
    cache.reserve("a", 1)
    t.fill(e)
    check_rows(t, cache, e)
    cache.commit("a", 1)
    first = list(cache.block_table(0, "a"))
    cache.release("a")
    cache.add_request("a")                             # the free list hands the pages back reversed
    cache.reserve("a", 21)
    cache.commit("a", 21)
    assert cache.block_table(0, "a") != first
    cache.reserve("a", 1)
    t.fill(e)
    check_rows(t, cache, e)


def test_a_shorter_request_takes_over_a_row():
    cache = CacheManager([(0, True, FULL, None)], 8, 16, 2)
    t = DecodeTables(cache, 2, 64)
    cache.add_request("long")
    cache.reserve("long", 41)
    cache.commit("long", 40)
    t.fill([StepEntry("long", [1], [0])])
    cache.commit("long", 1)
    cache.add_request("short")
    cache.reserve("short", 4)
    cache.commit("short", 3)
    ents = [StepEntry("short", [2], [0]), StepEntry("long", [3], [0])]
    cache.reserve("long", 1)
    t.fill(ents)
    check_rows(t, cache, ents)
    row = t.block_table_row(0, 0)
    assert not np.any(row[1:])                         # nothing of the former tenant is left


def test_lives_are_unique():
    cache = CacheManager([(0, True, FULL, None)], 8, 4, 2)
    seen = set()
    for _ in range(5):
        for rid in ("x", "y"):
            cache.add_request(rid)
            assert cache.life(rid) not in seen
            seen.add(cache.life(rid))
        cache.release("x")
        cache.release("y")


def test_half_way_buckets_wait_for_their_capture_until_they_are_popular():
    """A decode step runs in the smallest bucket that holds it; where a graph of less than twice
    that bucket's rows exists already, it stands in until the bucket has been wanted often."""
    from types import SimpleNamespace
    from tffinfer_amd.engine.runner import ModelRunner
    assert graph_buckets(64) == [1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64]
    assert graph_buckets(20) == [1, 2, 3, 4, 6, 8, 12, 16, 20] and graph_buckets(1) == [1]
    r = SimpleNamespace(_graph_buckets=graph_buckets(64), _graphs={}, _graph_wanted={},
                        CAPTURE_AFTER=ModelRunner.CAPTURE_AFTER)
    pick = lambda n: ModelRunner._pick_bucket(r, n)
    assert pick(32) == 32                      # nothing captured yet: its own bucket, now
    r._graphs[32] = object()
    assert pick(20) == 32 and pick(17) == 32   # 24 is wanted, 32 stands in
    assert pick(16) == 16                      # 32 is twice 16: no stand-in
    r._graphs[16] = object()
    assert pick(12) == 16                      # 16 < 2 * 12 stands in for 12
    assert pick(5) == 6                        # 16 and 32 are more than twice 6
    for _ in range(ModelRunner.CAPTURE_AFTER - 3):
        assert pick(24) == 32
    assert pick(24) == 24                      # wanted often enough: captured now
    r._graphs[24] = object()
    assert pick(17) == 24 and r._graph_wanted[24] == ModelRunner.CAPTURE_AFTER
