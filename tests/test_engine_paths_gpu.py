"""The engine's faster paths against the plain implementation: decode graphs
through preemptions (a request that comes back to its graph row with other
pages), and decode steps launched ahead of the tokens of the step in flight
(with a request that ends on a stop token while a step is ahead, and one that
is aborted then).  Every kept row of logits is compared with the plain logits
of the engine's own sequence, and every chosen token with the plain sampler's
choice from that row."""
import pytest
import torch

from helpers import oracle_logits, random_tokens, read_config
from test_generate_gpu import check_choices

pytestmark = pytest.mark.gpu


def drive(eng, arrivals, on_step=None):
    """Steps the engine until nothing is left; ``arrivals`` maps a step number to the
    requests (keyword arguments of add_request) that arrive before it."""
    step = 0
    pending = dict(arrivals)
    while eng.has_work or pending:
        if not eng.has_work and step not in pending:
            step = min(pending)
        for kw in pending.pop(step, []):
            eng.add_request(**kw)
        if on_step:
            on_step(step)
        eng.step()
        eng.runner.cache.check()
        step += 1
        assert step < 2000


def watch_graph_rows(eng):
    """Counts the fills of a decode graph's row that find the same request id in the row but
    other pages than the request holds now: it went away and came back."""
    from tffinfer_amd.engine.graphs import DecodeTables
    seen = {"returns": 0, "fills": 0}
    inner = DecodeTables.fill

    def fill(self, entries):
        for r, e in enumerate(entries):
            prev = self._row_state[r]
            if prev is None or prev[0] != e.req:
                continue
            for gi, g in enumerate(self.cache.groups):
                n = min(prev[-1][gi], len(self.cache.block_table(gi, e.req)))
                if g.spec.window == 0 and list(self.block_table_row(gi, r)[:n]) != self.cache.block_table(gi, e.req)[:n]:
                    seen["returns"] += 1
        seen["fills"] += 1
        return inner(self, entries)

    return seen, fill


@pytest.mark.parametrize("name", ["A", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_preempted_request_decodes_again_in_its_graph_row(model_dirs, dtype, name, monkeypatch):
    """Three requests arrive one after the other on 11 pages of 8 tokens; the newest is
    preempted while it decodes, computed again and decodes again in the graph row it had,
    beside the same neighbours, with pages in another order."""
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    from tffinfer_amd.engine.graphs import DecodeTables
    d = model_dirs[name]
    V = read_config(d)["vocab_size"]
    lens, new, arrive = [12, 9, 26], [55, 36, 53], [0, 34, 19]
    sc = [SamplingConfig(), SamplingConfig("random", temperature=0.8, seed=77), SamplingConfig()]
    opt = EngineOptions(dtype=dtype, page_size=8, num_pages=11, max_num_seqs=3, max_num_batched_tokens=48,
                        prefill_chunk=24, max_model_len=128, use_graphs=True, run_ahead=False)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True
    seen, fill = watch_graph_rows(eng)
    monkeypatch.setattr(DecodeTables, "fill", fill)
    arrivals = {}
    for i in range(3):
        arrivals.setdefault(arrive[i], []).append(dict(
            prompt_ids=random_tokens(lens[i], V, 300 + i), sampling=sc[i], max_new_tokens=new[i],
            ignore_eos=True, request_id=i))
    drive(eng, arrivals)
    assert eng.scheduler.stats.preemptions > 0
    assert seen["returns"] > 0, "no request came back to its row: the schedule misses the case"
    for i in range(3):
        r = eng.pop_result(i)
        assert len(r.output) == new[i]
        check_choices(d, r, dtype, sc[i])
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_request_id_freed_and_used_again_on_a_graph_runner(model_dirs, dtype):
    """At the step function's level: a request decodes through the graph, is freed, the same id
    is added again while another request holds pages in between, and decodes again."""
    from tffinfer_amd.engine import ModelRunner, StepEntry
    from tffinfer_amd.models import load_model
    from helpers import rel_err, tol
    d = model_dirs["A"]
    V = read_config(d)["vocab_size"]
    model = load_model(d, torch.float32 if dtype == "float32" else torch.bfloat16, "cuda:0")
    rn = ModelRunner(model, page_size=8, num_pages=12, max_seqs=2, max_model_len=96, use_graphs=True)

    def life(rid, toks, n_whole):
        ref = oracle_logits(d, toks)
        rn.add_request(rid)
        out = rn.step([StepEntry(rid, toks[:n_whole], [n_whole - 1])])
        assert rel_err(out[0], ref[n_whole - 1]) <= tol(dtype, "A")
        for j in range(n_whole, len(toks)):
            out = rn.step([StepEntry(rid, [toks[j]], [0])])       # one token: the graph
            assert rel_err(out[0], ref[j]) <= tol(dtype, "A"), (rid, j)
        rn.cache.check()

    first = random_tokens(40, V, 401)
    life("a", first, 20)
    rn.add_request("b")
    rn.step([StepEntry("b", random_tokens(5, V, 402), [])])        # holds a page of its own
    rn.free_request("a")
    rn.step([StepEntry("b", random_tokens(9, V, 403), [])])        # and takes one of a's
    life("a", random_tokens(40, V, 404), 34)                       # same id, as many pages, other ones
    rn.free_request("a")
    rn.free_request("b")
    assert all(g.pool.num_used == 0 for g in rn.cache.groups)


@pytest.mark.parametrize("dtype,use_graphs", [("float32", True), ("bfloat16", True), ("bfloat16", False),
                                              ("float32", False)])
def test_steps_launched_ahead_against_the_plain_implementation(model_dirs, dtype, use_graphs):
    """Steps launched ahead, with kept logits: six requests of different lengths on four slots and a
    pool that runs out; then the same with one request that stops on a token of its own choosing
    while a step is ahead, and one that is aborted while a step is ahead."""
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    d = model_dirs["B"]
    V = read_config(d)["vocab_size"]
    prompts = [random_tokens(n, V, 170 + n) for n in (3, 17, 31, 9, 26, 5)]
    sc = [SamplingConfig("random", temperature=0.7, seed=30 + i) if i % 2 else SamplingConfig() for i in range(6)]
    lens = [24, 7, 30, 16, 1, 21]
    opt = EngineOptions(dtype=dtype, page_size=8, num_pages=24, max_num_seqs=4, max_num_batched_tokens=48,
                        prefill_chunk=24, run_ahead=True, use_graphs=use_graphs)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True

    def requests(eos_for_2=None):
        return {0: [dict(prompt_ids=p, sampling=s, max_new_tokens=n, request_id=i,
                         ignore_eos=not (i == 2 and eos_for_2 is not None),
                         eos_token_id=eos_for_2 if i == 2 else None)
                    for i, (p, s, n) in enumerate(zip(prompts, sc, lens))]}

    drive(eng, requests())
    assert eng.steps_ahead > 10
    first = {}
    for i in range(6):
        r = first[i] = eng.pop_result(i)
        assert len(r.output) == lens[i] and r.finish_reason == "length"
        check_choices(d, r, dtype, sc[i])
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)

    # request 2 stops at the token it chose as its 12th; request 0 is aborted while a step is ahead
    eos = first[2].output[11]
    aborted = {}

    def on_step(step):
        req0 = eng._requests.get(0)
        if not aborted and eng._ahead is not None and req0 is not None and len(req0.output) >= 9:
            assert any(p.request.id == 0 for p in eng._ahead.plan)    # a token of its is in flight
            assert eng.abort(0)
            aborted["at"] = len(req0.output)

    before = eng.steps_ahead
    drive(eng, requests(eos), on_step)
    assert eng.steps_ahead > before + 10 and aborted
    for i in range(6):
        r = eng.pop_result(i)
        if i == 0:
            assert r.finish_reason == "abort" and len(r.output) == aborted["at"]
            if dtype == "float32":     # the same choices whoever else is in the batch
                assert r.output == first[0].output[:aborted["at"]]
        elif i == 2:
            assert r.finish_reason == "stop" and r.output[-1] == eos and eos not in r.output[:-1]
            if dtype == "float32":
                assert r.output == first[2].output[:first[2].output.index(eos) + 1]
        else:
            assert r.finish_reason == "length" and len(r.output) == lens[i]
        assert len(r.logits) == len(r.output)
        check_choices(d, r, dtype, sc[i])
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
    assert eng.runner.cache.slots.num_free == 4


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("D", "bfloat16"), ("D", "float32"), ("A", "bfloat16")])
def test_random_workloads_on_small_pools(model_dirs, name, dtype, seed):
    """Random workloads (lengths, arrival steps, sampling, stop lengths, an abort) on pools that
    hold about half of what the requests need together, with decode graphs and steps launched
    ahead: whatever the schedule turns out to be (admissions, portions, preemptions, windows that
    give pages back, rows that change hands), every kept row of logits matches the plain logits
    of the request's own sequence and every token is the plain sampler's choice."""
    import random
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    rng = random.Random(1000 * seed + 17 * ord(name) + (7 if dtype == "float32" else 0))
    d = model_dirs[name]
    cfg = read_config(d)
    V, limit = cfg["vocab_size"], min(cfg["max_position_embeddings"], 160)
    n = rng.randrange(3, 7)
    ps = rng.choice([8, 16])
    reqs, need = [], 0
    for i in range(n):
        plen, new = rng.randrange(1, 60), rng.randrange(2, 45)
        new = min(new, limit - plen - 1)
        sc = SamplingConfig("random", temperature=rng.choice([0.6, 1.0, 1.3]), seed=rng.randrange(1 << 20)) \
            if rng.random() < 0.5 else SamplingConfig()
        reqs.append(dict(prompt_ids=random_tokens(plen, V, 7000 + 31 * seed + i), sampling=sc, max_new_tokens=new,
                         ignore_eos=True, request_id=i))
        need += -(-(plen + new) // ps)
    biggest = max(-(-(len(r["prompt_ids"]) + r["max_new_tokens"]) // ps) for r in reqs)
    pages = max(biggest + 1, need // 2)
    slots = rng.randrange(2, 5)
    opt = EngineOptions(dtype=dtype, page_size=ps, num_pages=pages, max_num_seqs=slots,
                        max_num_batched_tokens=rng.choice([16, 32, 64]), prefill_chunk=rng.choice([8, 16, 24]),
                        max_model_len=limit, use_graphs=True, run_ahead=True)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True
    arrivals = {}
    for r in reqs:
        arrivals.setdefault(rng.randrange(0, 40), []).append(r)
    victim = rng.randrange(n) if rng.random() < 0.5 else None
    state = {}

    def on_step(step):
        r = eng._requests.get(victim)
        if victim is not None and "done" not in state and r is not None and r.status == "running" and len(r.output) >= 2:
            eng.abort(victim)
            state["done"] = True

    drive(eng, arrivals, on_step)
    st = eng.scheduler.stats
    print(f"{name} {dtype} seed {seed}: {n} requests, {pages} pages of {ps}, {slots} slots: {st.steps} steps, "
          f"{st.preemptions} preemptions, {eng.steps_ahead} steps launched ahead, {len(eng.runner._graphs)} graphs")
    for r in reqs:
        res = eng.pop_result(r["request_id"])
        if res.finish_reason == "abort":
            assert r["request_id"] == victim
        else:
            assert res.finish_reason == "length" and len(res.output) == r["max_new_tokens"]
        assert len(res.logits) == len(res.output)
        check_choices(d, res, dtype, r["sampling"])
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
    assert eng.runner.cache.slots.num_free == slots


@pytest.mark.parametrize("use_graphs", [False, True])
def test_a_step_that_fails_gives_its_pages_back(model_dirs, use_graphs, monkeypatch):
    """A step that raises after its pages were taken (a kernel that refuses its operands, memory
    that runs out) leaves the cache as it found it: the pages go back, the requests keep their
    counts, and the same step runs afterwards as if nothing had happened."""
    from tffinfer_amd.engine import ModelRunner, StepEntry
    from tffinfer_amd.engine.graphs import DecodeGraph
    from tffinfer_amd.kernels import lib, ops
    from tffinfer_amd.models import load_model
    from helpers import rel_err, tol
    d = model_dirs["A"]
    V = read_config(d)["vocab_size"]

    class Failing:
        armed = 0

        def __getattr__(self, name):
            real = getattr(ops, name)
            if name != "linear":
                return real

            def linear(*a, **kw):
                if self.armed:
                    self.armed -= 1
                    if self.armed == 0:
                        raise lib.KernelError("made to fail")
                return real(*a, **kw)
            return linear

    stub = Failing()
    model = load_model(d, torch.float32, "cuda:0")
    rn = ModelRunner(model, page_size=8, num_pages=12, max_seqs=2, max_model_len=96, use_graphs=use_graphs, ops=stub)
    a, b = random_tokens(40, V, 501), random_tokens(12, V, 502)
    ref_a, ref_b = oracle_logits(d, a), oracle_logits(d, b)
    rn.add_request("a")
    rn.add_request("b")
    rn.step([StepEntry("a", a[:5], [])])
    used = [g.pool.num_used for g in rn.cache.groups]
    stub.armed = 3                                          # the third product of the step raises
    with pytest.raises(lib.KernelError, match="made to fail"):
        rn.step([StepEntry("a", a[5:32], [26]), StepEntry("b", b[:11], [10])])
    assert [g.pool.num_used for g in rn.cache.groups] == used
    assert rn.cache.num_tokens("a") == 5 and rn.cache.num_tokens("b") == 0
    rn.cache.check()
    out = rn.step([StepEntry("a", a[5:32], [26]), StepEntry("b", b[:11], [10])])
    assert rel_err(out[0], ref_a[31]) <= tol("float32", "A") and rel_err(out[1], ref_b[10]) <= tol("float32", "A")
    # a decode step (through the graph, where there is one) that fails before anything ran
    used = [g.pool.num_used for g in rn.cache.groups]
    if use_graphs:
        inner = DecodeGraph.run
        state = {"fail": True}

        def run(self, entries, token_source=None):
            if state.pop("fail", False):
                raise RuntimeError("made to fail")
            return inner(self, entries, token_source)
        monkeypatch.setattr(DecodeGraph, "run", run)
    else:
        stub.armed = 2
    with pytest.raises((RuntimeError, lib.KernelError), match="made to fail"):
        rn.step([StepEntry("a", [a[32]], [0]), StepEntry("b", [b[11]], [0])])      # a's token opens a new page
    assert [g.pool.num_used for g in rn.cache.groups] == used and rn.cache.num_tokens("a") == 32
    out = rn.step([StepEntry("a", [a[32]], [0]), StepEntry("b", [b[11]], [0])])
    assert rel_err(out[0], ref_a[32]) <= tol("float32", "A") and rel_err(out[1], ref_b[11]) <= tol("float32", "A")
    rn.free_request("a")
    rn.free_request("b")
    assert all(g.pool.num_used == 0 for g in rn.cache.groups)


@pytest.mark.parametrize("run_ahead", [False, True])
def test_the_engine_goes_on_after_a_step_that_failed(model_dirs, run_ahead):
    """A product refuses its operands in the middle of a prompt step, and again in a decode step
    (launched ahead of the tokens of the step in flight, where that is on): step() raises, and
    the engine, stepped on, gives every request the tokens of an undisturbed run."""
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    from tffinfer_amd.kernels import lib, ops
    d = model_dirs["A"]
    V = read_config(d)["vocab_size"]
    prompts = [random_tokens(n, V, 640 + n) for n in (30, 7, 19)]
    sc = [SamplingConfig(), SamplingConfig("random", temperature=0.8, seed=3), SamplingConfig()]

    class Failing:
        calls, fail_at = 0, set()

        def __getattr__(self, name):
            real = getattr(ops, name)
            if name != "linear":
                return real

            def linear(*a, **kw):
                self.calls += 1
                if self.calls in self.fail_at:
                    raise lib.KernelError("made to fail")
                return real(*a, **kw)
            return linear

    def run(fail_at):
        opt = EngineOptions(dtype="float32", page_size=8, num_pages=40, max_num_seqs=3, max_num_batched_tokens=32,
                            prefill_chunk=16, use_graphs=False, run_ahead=run_ahead)
        eng = LLMEngine.from_model_dir(d, opt)
        stub = Failing()
        stub.fail_at = set(fail_at)
        eng.runner.ops = stub
        eng.keep_logits = True
        ids = [eng.add_request(p, s, max_new_tokens=12, ignore_eos=True) for p, s in zip(prompts, sc)]
        errors = 0
        while eng.has_work:
            try:
                eng.step()
            except lib.KernelError:
                errors += 1
            eng.runner.cache.check()
        assert errors == len(fail_at)
        res = [eng.pop_result(i) for i in ids]
        assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
        return res, stub.calls

    clean, calls = run(())
    # the tenth product lies in the first steps (prompts), one near the end in a decode step
    broken, _ = run((10, calls - 40))
    for a, b, s in zip(clean, broken, sc):
        assert a.output == b.output and len(b.output) == 12
        check_choices(d, b, "float32", s)
