"""The scheduler's decisions on the host, with a stand-in for the step function
that commits tokens to the cache manager and picks the next token as a function
of everything the request has been fed so far (so a recomputation after a
preemption that fed wrong tokens would show)."""
import pytest

from tffinfer_amd.cache import CacheManager
from tffinfer_amd.engine.scheduler import Request, RequestRefused, Scheduler, SchedulerOptions
from tffinfer_amd.parts.base import KVCacheSpec
from tffinfer_amd.sampling import SamplingConfig

SPEC = KVCacheSpec(2, 16, 0)
WIN = KVCacheSpec(2, 16, 16)


class FakeRunner:
    def __init__(self, cache):
        self.cache = cache
        self.fed = {}        # request id -> tokens fed since its (re)admission

    def run(self, plan):
        sampled = {}
        for p in plan:
            rid = p.request.id
            if self.cache.num_tokens(rid) == 0:
                self.fed[rid] = []
            assert p.start == self.cache.num_tokens(rid) == len(self.fed[rid])
            toks = p.request.tokens[p.start:p.start + p.count]
            assert len(toks) == p.count
            self.fed[rid].extend(toks)
            self.cache.commit(rid, p.count)
            if p.samples:
                assert len(self.fed[rid]) == len(p.request.tokens)
                sampled[rid] = next_token(self.fed[rid])
        return sampled


def next_token(tokens):
    h = 17
    for t in tokens:
        h = (h * 31 + t + 1) % 1009
    return h % 97


def expected_output(prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(next_token(toks))
    return toks[len(prompt):]


def make(num_pages=64, ps=8, max_seqs=4, budget=64, chunk=24, max_len=512, specs=(SPEC,)):
    cache = CacheManager([(i, True, s, None) for i, s in enumerate(specs)], ps, num_pages, max_seqs)
    sched = Scheduler(cache, SchedulerOptions(max_seqs, budget, chunk), max_len)
    return cache, sched, FakeRunner(cache)


def run_all(sched, runner, cache, limit=5000, on_step=None):
    steps = 0
    while sched.has_work:
        plan = sched.schedule()
        assert plan, "work left but nothing scheduled"
        if on_step:
            on_step(plan)
        sched.update(plan, runner.run(plan))
        cache.check()
        steps += 1
        assert steps < limit
    return steps


def test_portions_budget_and_decode_first():
    cache, sched, runner = make(budget=40, chunk=24)
    reqs = [Request(i, list(range(1, n + 1)), max_new_tokens=6) for i, n in enumerate([3, 50, 31])]
    for r in reqs:
        sched.add_request(r)
    seen_mixed = []

    def on_step(plan):
        total = sum(p.count for p in plan)
        assert total <= 40
        ids = [p.request.id for p in plan]
        assert len(ids) == len(set(ids))
        decodes = [p for p in plan if p.request.num_pending == 1]
        if any(p.start > 0 for p in decodes):       # somebody decodes: no portion beyond the chunk
            assert all(p.count <= 24 for p in plan)
        if decodes:  # decodes come first in the plan and are never left out
            assert plan[:len(decodes)] == decodes
            running_decoding = [r for r in sched.running if r.num_pending == 1]
            assert len(decodes) == len(running_decoding)
        if decodes and len(decodes) < len(plan):
            seen_mixed.append(True)

    run_all(sched, runner, cache, on_step=on_step)
    assert seen_mixed, "no step mixed a prompt portion with decode tokens"
    for r in reqs:
        assert r.status == "finished" and r.finish_reason == "length"
        assert r.output == expected_output(r.prompt, 6)
    assert cache.groups[0].pool.num_used == 0 and cache.slots.num_free == 4


def test_prompts_share_the_whole_budget_while_nobody_decodes():
    """The chunk bounds a step's time for the sake of requests that decode in it.  A prompt alone
    takes the whole budget; two prompts take a chunk each and the first what is left; beside a
    request that decodes no portion is longer than the chunk."""
    cache, sched, runner = make(budget=64, chunk=24)
    sched.add_request(Request("a", list(range(100)), max_new_tokens=3))
    plan = sched.schedule()
    assert [(p.request.id, p.start, p.count, p.samples) for p in plan] == [("a", 0, 64, False)]
    sched.update(plan, runner.run(plan))
    sched.add_request(Request("b", list(range(1, 81)), max_new_tokens=3))
    plan = sched.schedule()          # 36 tokens of a are left: its chunk, b's chunk, the rest of a; 4 more for b
    assert [(p.request.id, p.start, p.count, p.samples) for p in plan] == [("a", 64, 36, True), ("b", 0, 28, False)]
    sched.update(plan, runner.run(plan))
    plan = sched.schedule()          # a decodes now: b gets a chunk and no more
    assert [(p.request.id, p.start, p.count, p.samples) for p in plan] == [("a", 100, 1, True), ("b", 28, 24, False)]
    sched.update(plan, runner.run(plan))
    run_all(sched, runner, cache)
    assert cache.groups[0].pool.num_used == 0


def test_leftover_budget_is_bounded_by_free_pages():
    """What is left of the budget goes to a prompt only as far as pages are free."""
    cache, sched, runner = make(num_pages=6, ps=8, budget=64, chunk=16, max_len=64)
    sched.add_request(Request("a", list(range(47)), max_new_tokens=1))
    plan = sched.schedule()
    assert [(p.request.id, p.start, p.count, p.samples) for p in plan] == [("a", 0, 47, True)]
    sched.update(plan, runner.run(plan))
    cache2, sched2, runner2 = make(num_pages=6, ps=8, budget=64, chunk=16, max_len=64)
    sched2.add_request(Request("x", list(range(30)), max_new_tokens=1))
    sched2.add_request(Request("y", list(range(30)), max_new_tokens=1))
    plan = sched2.schedule()         # six pages of eight: 30 tokens take four, 16 take two, nothing is left for more
    assert [(p.request.id, p.count) for p in plan] == [("x", 30), ("y", 16)]
    sched2.update(plan, runner2.run(plan))
    cache2.check()


def test_admission_in_arrival_order_and_slot_limit():
    cache, sched, runner = make(max_seqs=2, budget=64, chunk=16)
    for i in range(4):
        sched.add_request(Request(i, [5] * 10, max_new_tokens=3))
    plan = sched.schedule()
    assert [p.request.id for p in plan] == [0, 1]
    assert [r.id for r in sched.waiting] == [2, 3]
    order = []
    sched.update(plan, runner.run(plan))
    run_all(sched, runner, cache, on_step=lambda plan: order.extend(p.request.id for p in plan if p.start == 0))
    assert order == [2, 3]


def test_eos_and_length_finish():
    cache, sched, runner = make()
    prompt = [1, 2, 3]
    out = expected_output(prompt, 10)
    r1 = Request("e", list(prompt), max_new_tokens=10, eos_token_id=out[3])
    r2 = Request("i", list(prompt), max_new_tokens=10, eos_token_id=out[3], ignore_eos=True)
    sched.add_request(r1)
    sched.add_request(r2)
    run_all(sched, runner, cache)
    assert r1.finish_reason == "stop" and r1.output == out[:out.index(out[3]) + 1]
    assert r2.finish_reason == "length" and r2.output == out


def test_refused_requests():
    cache, sched, _ = make(num_pages=4, ps=8, max_len=64)
    with pytest.raises(RequestRefused, match="length limit"):
        sched.add_request(Request("long", [1] * 60, max_new_tokens=10))
    with pytest.raises(RequestRefused, match="cache pages"):
        sched.add_request(Request("big", [1] * 40, max_new_tokens=2))   # 41 tokens need 6 pages of 4
    with pytest.raises(RequestRefused, match="empty"):
        sched.add_request(Request("none", [], max_new_tokens=2))
    sched.add_request(Request("fits", [1] * 20, max_new_tokens=13))     # 32 tokens in the cache: 4 pages
    assert len(sched.waiting) == 1


def test_pages_run_out_preempts_the_newest_and_outputs_stay_equal():
    # each request alone fits (<= 6 pages), all together need far more than the 8 there are
    cache, sched, runner = make(num_pages=8, ps=8, max_seqs=4, budget=32, chunk=16)
    reqs = [Request(i, [(7 * i + j) % 50 for j in range(n)], max_new_tokens=20)
            for i, n in enumerate([20, 9, 26, 14, 5])]
    for r in reqs:
        sched.add_request(r)
    preempted_newest = []
    orig = sched._preempt_last

    def spy():
        newest = sched.running[-1]
        v = orig()
        preempted_newest.append(v is newest)
        assert sched.waiting[0] is v and v.num_computed == 0 and not cache.has_request(v.id)
        return v

    sched._preempt_last = spy
    run_all(sched, runner, cache)
    assert sched.stats.preemptions > 0 and all(preempted_newest)
    for r in reqs:
        assert r.output == expected_output(r.prompt, 20), f"request {r.id} changed by preemption"
    assert sum(r.num_preemptions for r in reqs) == sched.stats.preemptions
    assert cache.groups[0].pool.num_used == 0


def test_oldest_request_is_never_preempted_while_others_run():
    cache, sched, runner = make(num_pages=6, ps=8, max_seqs=3, budget=32, chunk=16)
    reqs = [Request(i, [i + 1] * 12, max_new_tokens=30) for i in range(3)]
    for r in reqs:
        sched.add_request(r)
    run_all(sched, runner, cache)
    assert reqs[0].num_preemptions == 0
    assert all(r.output == expected_output(r.prompt, 30) for r in reqs)


def test_window_group_needs_fewer_pages():
    cache, sched, runner = make(num_pages=6, ps=8, max_seqs=2, budget=16, chunk=8, specs=(WIN,))
    # 100 tokens would need 13 pages in a full group; the window of 16 needs 4 at most
    r = Request("w", list(range(80)), max_new_tokens=20)
    sched.add_request(r)
    run_all(sched, runner, cache, on_step=lambda plan: None)
    assert r.output == expected_output(r.prompt, 20) and sched.stats.preemptions == 0


def test_abort():
    cache, sched, runner = make()
    sched.add_request(Request("a", [1] * 30, max_new_tokens=5))
    sched.add_request(Request("b", [2] * 30, max_new_tokens=5))
    plan = sched.schedule()
    sched.update(plan, runner.run(plan))
    assert sched.abort("a") and not sched.abort("zzz")
    assert not cache.has_request("a")
    run_all(sched, runner, cache)
    assert cache.groups[0].pool.num_used == 0


def test_stats_and_determinism():
    outs = []
    for _ in range(2):
        cache, sched, runner = make(num_pages=10, budget=24, chunk=8)
        reqs = [Request(i, [i] * (5 + 3 * i), max_new_tokens=7) for i in range(5)]
        for r in reqs:
            sched.add_request(r)
        trace = []
        run_all(sched, runner, cache, on_step=lambda plan: trace.append([(p.request.id, p.start, p.count) for p in plan]))
        outs.append(trace)
        assert sched.stats.finished == 5 and sched.stats.steps == len(trace)
    assert outs[0] == outs[1]


def test_seen_tokens_keep_up_with_a_growing_sequence():
    """The distinct tokens a repetition penalty needs, brought up to date token by token, are
    those of the whole sequence at every length, each once."""
    import random
    import numpy as np
    from tffinfer_amd.sampling import SeenTokens
    rnd = random.Random(4)
    seq = [rnd.randrange(40) for _ in range(30)]
    seen = SeenTokens()
    assert seen.update([]).size == 0
    for n in (1, 2, 2, 9, 30):
        got = seen.update(seq[:n])
        assert got.dtype == np.int32 and sorted(got.tolist()) == sorted(set(seq[:n])) and len(set(got.tolist())) == got.size
    for _ in range(700):              # beyond the first buffer
        seq.append(rnd.randrange(5000))
    assert sorted(seen.update(seq).tolist()) == sorted(set(seq))


def test_sampling_config_validation():
    with pytest.raises(ValueError):
        SamplingConfig(type="unknown")
    with pytest.raises(ValueError):
        SamplingConfig(top_p=0.0)
    assert SamplingConfig().greedy and SamplingConfig("default").greedy
    assert SamplingConfig("random", temperature=0.0).greedy
    assert SamplingConfig("top_k", 0.7, top_k=5).effective() == (0.7, 5, 1.0, 0.0)


def test_a_head_of_the_queue_that_fits_nowhere_is_finished_not_raised():
    """Pages held by somebody the scheduler does not know (so that its own check at
    add_request passes): the head cannot get a single token even with nothing running.  It is
    taken out and finished as "refused"; the requests behind it run once pages are there."""
    cache, sched, runner = make(num_pages=4, ps=8)
    cache.add_request("elsewhere")
    cache.reserve("elsewhere", 32)                    # every page
    a, b = Request("a", [1] * 5, max_new_tokens=3), Request("b", [2] * 5, max_new_tokens=3)
    sched.add_request(a)
    assert sched.schedule() == []
    assert a.status == "finished" and a.finish_reason == "refused" and sched.refused == [a]
    assert not sched.has_work
    cache.release("elsewhere")
    sched.add_request(b)
    run_all(sched, runner, cache)
    assert b.output == expected_output(b.prompt, 3)


def test_window_group_of_the_least_size_runs_under_a_large_budget():
    """A window of 16 in pages of 8 needs ceil(15 / 8) + 1 = 3 pages to advance by a token.  On
    exactly that pool a long request is admitted and runs to its end although the token budget
    would let its portions grow to 64 tokens: portions are cut to what the free pages hold."""
    from tffinfer_amd.cache.sizing import min_window_pages
    assert min_window_pages(16, 8) == 3
    cache, sched, runner = make(num_pages=3, ps=8, max_seqs=1, budget=64, chunk=24, specs=(WIN,))
    r = Request("w", list(range(90)), max_new_tokens=20)
    sched.add_request(r)
    sizes = []
    run_all(sched, runner, cache, on_step=lambda plan: sizes.append(plan[0].count))
    assert r.output == expected_output(r.prompt, 20) and sched.stats.preemptions == 0
    assert max(sizes) <= 3 * 8 and max(sizes) > 1
    # one page fewer and the request can never advance past its window: refused when added
    cache, sched, runner = make(num_pages=2, ps=8, max_seqs=1, budget=64, chunk=24, specs=(WIN,))
    with pytest.raises(RequestRefused, match="cache pages"):
        sched.add_request(Request("w", list(range(90)), max_new_tokens=20))
    # a short one that fits its two pages whole is taken
    sched.add_request(Request("s", list(range(10)), max_new_tokens=5))
    run_all(sched, runner, cache)


def test_window_pool_sized_by_the_engine_never_preempts():
    """Pools as the engine sizes them: the group that keeps all keys holds every request, the
    group with a window gets window_pool_pages; four long requests run under a budget that a lone
    prompt may fill, and nothing is ever preempted for want of a window page."""
    from tffinfer_amd.cache.sizing import plan_pages
    ps, seqs, budget = 8, 4, 64
    reqs_spec = [(0, True, SPEC, None), (1, True, WIN, None)]
    pages = plan_pages(reqs_spec, ps, 2, seqs, budget, tokens=4 * 200)
    assert pages[WIN] < pages[SPEC] // 4
    cache = CacheManager(reqs_spec, ps, pages, seqs)
    sched = Scheduler(cache, SchedulerOptions(seqs, budget, 24), 512)
    runner = FakeRunner(cache)
    reqs = [Request(i, [(3 * i + j) % 60 for j in range(n)], max_new_tokens=40)
            for i, n in enumerate([150, 90, 30, 120, 77, 140])]
    for r in reqs:
        sched.add_request(r)
    run_all(sched, runner, cache)
    assert sched.stats.preemptions == 0
    assert all(r.output == expected_output(r.prompt, 40) for r in reqs)


def test_a_step_a_little_over_a_multiple_of_the_quantum_is_cut_down_to_it():
    """A quantum of 64 tokens: a portion of 64 beside 5 decoding requests makes 69 rows, a tile
    row more than 64; the portion is cut to 59.  A prompt's last portion is never cut (its first
    token would come a step later), nor is anything cut when the excess is more than a quarter
    of the quantum, or when the step is below one quantum."""
    cache = CacheManager([(0, True, SPEC, None)], 8, 200, 8)
    sched = Scheduler(cache, SchedulerOptions(8, 256, 64, token_quantum=64), 1024)
    runner = FakeRunner(cache)
    short = [Request(i, [i + 1] * 3, max_new_tokens=40) for i in range(5)]
    for r in short:
        sched.add_request(r)
    plan = sched.schedule()                      # five short prompts: 15 tokens, below a quantum
    assert sum(p.count for p in plan) == 15
    sched.update(plan, runner.run(plan))
    long = Request("long", list(range(300)), max_new_tokens=8)
    sched.add_request(long)
    seen = []
    while long.num_computed < 300:
        plan = sched.schedule()
        total = sum(p.count for p in plan)
        portion = next(p for p in plan if p.request is long)
        seen.append((total, portion.count, portion.samples))
        sched.update(plan, runner.run(plan))
        cache.check()
    # 5 decodes + 64 = 69 -> 64 (59 of the prompt), four times; then the 64 tokens that are left: the
    # prompt's last portion, uncut although 5 + 64 = 69 again
    assert seen == [(64, 59, False)] * 4 + [(69, 64, True)]
    run_all(sched, runner, cache)
    assert long.output == expected_output(long.prompt, 8)
    assert all(r.output == expected_output(r.prompt, 40) for r in short)
    assert cache.groups[0].pool.num_used == 0
    # an excess of more than a quarter of the quantum stays: 20 decodes + 64
    cache = CacheManager([(0, True, SPEC, None)], 8, 400, 24)
    sched = Scheduler(cache, SchedulerOptions(24, 256, 64, token_quantum=64), 1024)
    runner = FakeRunner(cache)
    for i in range(20):
        sched.add_request(Request(i, [i + 1] * 2, max_new_tokens=30))
    plan = sched.schedule()
    sched.update(plan, runner.run(plan))
    sched.add_request(Request("long", list(range(200)), max_new_tokens=4))
    plan = sched.schedule()
    assert sum(p.count for p in plan) == 84 and any(p.count == 64 for p in plan)
    # and pages taken for the tokens cut away went back
    cache = CacheManager([(0, True, SPEC, None)], 8, 50, 4)
    sched = Scheduler(cache, SchedulerOptions(4, 256, 64, token_quantum=64), 1024)
    runner = FakeRunner(cache)
    for i in range(3):
        sched.add_request(Request(i, [i + 1], max_new_tokens=30))
    plan = sched.schedule()
    sched.update(plan, runner.run(plan))
    sched.add_request(Request("long", list(range(200)), max_new_tokens=4))
    plan = sched.schedule()
    assert sorted(p.count for p in plan) == [1, 1, 1, 61]
    assert len(cache.block_table(0, "long")) == 8        # 61 tokens: eight pages of 8, not the nine of 64
    cache.check()
