"""Decode steps of twenty and more requests through the engine, against the plain
implementation: the schedules that large batches take and small ones never reach.

With eight kv heads, twenty to thirty-two requests are 160 to 256 (request, kv head) pairs,
between which a decode step gives every request, if they are of about one length, a block of eight
waves per kv head instead of single waves per run of keys; products of 17 to 64 rows run on tiles whose blocks split K, with their partial sums added
up by the norm that follows or by a kernel of their own; and the batch shrinks through the graph
buckets 28, 24, 16, 12, 8, ... with a larger graph standing in for a smaller one on the way.  One
request many times longer than the others is cut into many runs of keys, whose partial results a
second kernel merges, while the short ones are a run each.  All of that runs inside captured HIP graphs with padding rows and with
steps launched ahead.  Every kept row of logits is compared with the plain logits of the
request's own sequence and every token with the plain sampler's choice from that row
(``check_choices``).
"""
import pytest
import torch

from helpers import random_tokens, read_config
from test_engine_paths_gpu import drive
from test_generate_gpu import check_choices

pytestmark = pytest.mark.gpu


def _watch(monkeypatch):
    """Records what the decode attention and the products were asked for."""
    from tffinfer_amd.kernels import ops
    seen = {"pairs": set(), "split_rows": set(), "stacks": set(), "blocks": set(), "merge": set()}
    inner_attn, inner_linear = ops.attention_decode_fused, ops.linear

    def attn(qkv, nq, nkv, *a, **kw):
        seen["pairs"].add(qkv.shape[0] * nkv)
        assert kw.get("key_runs") is not None, "a decode step without runs of keys"
        seen["blocks"].add(bool(kw["runs_for_blocks"]))
        seen["merge"].add(bool(kw["runs_merge"]))
        return inner_attn(qkv, nq, nkv, *a, **kw)

    def linear(x, weight, *a, **kw):
        out = inner_linear(x, weight, *a, **kw)
        if isinstance(out, torch.Tensor) and out.dim() == 3:
            seen["stacks"].add((out.shape[1], out.shape[0]))     # (rows, parts of K kept for the norm)
        return out

    monkeypatch.setattr(ops, "attention_decode_fused", attn)
    monkeypatch.setattr(ops, "linear", linear)
    return seen


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page_size", [("E", 16), ("W", 16), ("W", 64), ("W", 128)])
def test_twenty_eight_requests_shrinking_through_the_graph_buckets(model_dirs, name, page_size, dtype, monkeypatch):
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.kernels import ops
    d = model_dirs[name]
    cfg = read_config(d)
    V, nkv = cfg["vocab_size"], cfg["num_key_value_heads"]
    n = 28
    seen = _watch(monkeypatch)
    # a smaller bucket's graph is captured after it has been wanted three times; until then a
    # larger one stands in for it
    monkeypatch.setattr(ModelRunner, "CAPTURE_AFTER", 3)
    # prompts of 3 .. 140 tokens (pages of 128: some requests cross into a second page while they
    # decode, most live in a part of one); a request ends after 7 + 3 i tokens, so that the batch
    # loses one request every third step
    # (with pages of 64: prompts of about one length, for which twenty to twenty-eight requests get a
    # block of eight waves per request and kv head, padding rows beside them)
    even = page_size == 64
    plens = [100 + (7 * i) % 20 if even else 3 + (37 * i) % 138 for i in range(n)]
    news = [7 + 3 * i for i in range(n)]
    sc = [SamplingConfig("random", temperature=0.9, seed=500 + i) if i % 3 == 1 else SamplingConfig()
          for i in range(n)]
    opt = EngineOptions(dtype=dtype, page_size=page_size, kv_tokens=n * 256, max_num_seqs=n,
                        max_num_batched_tokens=1024, prefill_chunk=256, max_model_len=256,
                        use_graphs=True, run_ahead=True)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True
    reqs = [dict(prompt_ids=random_tokens(plens[i], V, 9000 + i), sampling=sc[i], max_new_tokens=news[i],
                 ignore_eos=True, request_id=i) for i in range(n)]
    standins = []
    pick = ModelRunner._pick_bucket

    def picked(self, R):
        b = pick(self, R)
        want = next(x for x in self._graph_buckets if x >= R)
        if b != want:
            standins.append((R, b))
        return b

    monkeypatch.setattr(ModelRunner, "_pick_bucket", picked)
    drive(eng, {0: reqs})
    graphs = sorted(eng.runner._graphs)
    print(f"{name} {dtype} pages of {page_size}: {eng.scheduler.stats.steps} steps, {eng.steps_ahead} launched ahead, "
          f"graphs {graphs}, stand-ins {sorted(set(standins))}, attention pairs {sorted(seen['pairs'])}, "
          f"kept partial sums (rows, parts) {sorted(seen['stacks'])}")
    assert eng.steps_ahead > 40
    assert {28, 24, 16, 12, 8}.issubset(graphs), graphs
    assert standins, "no graph ever stood in for a smaller one"
    if dtype == "bfloat16":
        assert False in seen["blocks"] and (True in seen["blocks"] or not even), \
            "single waves should have run, and blocks of eight waves for the requests of about one length"
        assert any(17 <= rows <= 64 and parts > 1 for rows, parts in seen["stacks"]), \
            "no product of 17 to 64 rows kept partial sums for the norm"
    for i in range(n):
        r = eng.pop_result(i)
        assert r.finish_reason == "length" and len(r.output) == news[i]
        check_choices(d, r, dtype, sc[i])
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
    assert eng.runner.cache.slots.num_free == n


@pytest.mark.parametrize("seed", range(3))
@pytest.mark.parametrize("name,dtype", [("E", "bfloat16"), ("E", "float32"), ("W", "bfloat16")])
def test_random_workloads_of_many_requests_on_small_pools(model_dirs, name, dtype, seed):
    """Random workloads of eighteen to twenty-six requests on sixteen to twenty-four slots and a
    pool that holds some six tenths of what they need together (lengths, arrival steps,
    sampling, an abort), with decode graphs and steps launched ahead: batches grow and shrink through the
    buckets, requests are preempted out of large batches and come back, rows change hands.
    Whatever the schedule, every kept row of logits matches the plain logits of the request's
    own sequence and every token is the plain sampler's choice."""
    import random
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    from tffinfer_amd.engine.runner import ModelRunner
    rng = random.Random(2000 * seed + 13 * ord(name) + (5 if dtype == "float32" else 0))
    d = model_dirs[name]
    cfg = read_config(d)
    V, limit = cfg["vocab_size"], 200
    n = rng.randrange(18, 27)
    ps = rng.choice([16, 32])
    reqs, need = [], 0
    for i in range(n):
        plen, new = rng.randrange(1, 90), rng.randrange(2, 50)
        sc = SamplingConfig("random", temperature=rng.choice([0.6, 1.0, 1.3]), seed=rng.randrange(1 << 20)) \
            if rng.random() < 0.4 else SamplingConfig()
        reqs.append(dict(prompt_ids=random_tokens(plen, V, 8000 + 41 * seed + i), sampling=sc, max_new_tokens=new,
                         ignore_eos=True, request_id=i))
        need += -(-(plen + new) // ps)
    biggest = max(-(-(len(r["prompt_ids"]) + r["max_new_tokens"]) // ps) for r in reqs)
    pages = max(biggest + 1, int(need * (0.55, 0.62, 0.68)[seed % 3]))
    slots = rng.randrange(16, 25)
    opt = EngineOptions(dtype=dtype, page_size=ps, num_pages=pages, max_num_seqs=slots,
                        max_num_batched_tokens=rng.choice([64, 128, 256]), prefill_chunk=rng.choice([16, 48, 96]),
                        max_model_len=limit, use_graphs=True, run_ahead=True)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True
    ModelRunner.CAPTURE_AFTER, kept = 4, ModelRunner.CAPTURE_AFTER
    try:
        arrivals = {}
        for r in reqs:
            arrivals.setdefault(rng.randrange(0, 12), []).append(r)
        victim = rng.randrange(n)
        state = {}

        def on_step(step):
            r = eng._requests.get(victim)
            if "done" not in state and r is not None and r.status == "running" and len(r.output) >= 2:
                eng.abort(victim)
                state["done"] = True

        drive(eng, arrivals, on_step)
    finally:
        ModelRunner.CAPTURE_AFTER = kept
    st = eng.scheduler.stats
    print(f"{name} {dtype} seed {seed}: {n} requests, {pages} pages of {ps}, {slots} slots: {st.steps} steps, "
          f"{st.preemptions} preemptions, {eng.steps_ahead} steps launched ahead, graphs {sorted(eng.runner._graphs)}")
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


@pytest.mark.parametrize("n,graphs", [(12, True), (24, True), (24, False), (40, True)])
def test_a_long_request_among_short_ones(tmp_path, n, graphs, monkeypatch):
    """One request of two thousand tokens beside requests of a few dozen: the long one's keys are
    cut into runs of the short ones' measure and merged, the short ones are a run each; once the
    long request has ended no step merges anything, and a captured step then runs in a variant
    without the merging kernel: on single waves, or, with twenty-four requests of about one length,
    on blocks of eight.  Every row of logits against the plain implementation."""
    from helpers import TINY_E, make_model_dir
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    cfg = dict(TINY_E, max_position_embeddings=4096)
    d = make_model_dir(str(tmp_path / "E"), cfg, 61)
    V = cfg["vocab_size"]
    seen = _watch(monkeypatch)
    # (the short requests: 40 to 52 tokens, two steps of keys each, about one length)
    plens = [2000] + [33 + (5 * i) % 13 for i in range(1, n)]
    news = [6] + [14] * (n - 1)
    opt = EngineOptions(dtype="bfloat16", page_size=16, kv_tokens=2100 + n * 96, max_num_seqs=n,
                        max_num_batched_tokens=4096, prefill_chunk=2048, max_model_len=2100,
                        use_graphs=graphs, run_ahead=graphs)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True
    reqs = [dict(prompt_ids=random_tokens(plens[i], V, 700 + i), sampling=SamplingConfig(), max_new_tokens=news[i],
                 ignore_eos=True, request_id=i) for i in range(n)]
    drive(eng, {0: reqs})
    assert seen["merge"] == {True, False}
    assert seen["blocks"] == ({True, False} if n == 24 else {False})
    if graphs:
        g = eng.runner._graphs[n]
        want = {(True, (False,)), (False, (True,))} if n == 24 else {(True, (False,)), (False, (False,))}
        assert set(g._variants) == want, f"the variants of the step of {n} rows: {sorted(g._variants)}"
        assert want <= set(g.possible_variants())
    for i in range(n):
        r = eng.pop_result(i)
        assert r.finish_reason == "length" and len(r.output) == news[i]
        check_choices(d, r, "bfloat16", None)


@pytest.mark.parametrize("seed", range(2))
def test_random_workloads_of_long_and_short_requests(tmp_path, seed, monkeypatch):
    """Requests of twenty to twenty-five hundred tokens under continuous batching on a pool that
    holds a third of them, with decode graphs and steps launched ahead: the runs of keys
    change with every admission, end and preemption, the captured steps switch between their
    variants, prompt portions run beside requests that decode over long contexts.  Every kept row
    of logits against the plain implementation, every token the plain sampler's choice."""
    import random
    from helpers import TINY_E, make_model_dir
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    rng = random.Random(77 + seed)
    cfg = dict(TINY_E, max_position_embeddings=4096)
    d = make_model_dir(str(tmp_path / "E"), cfg, 62 + seed)
    V = cfg["vocab_size"]
    seen = _watch(monkeypatch)
    n, ps = 12, 16
    reqs, need = [], 0
    for i in range(n):
        plen = rng.choice([rng.randrange(20, 200), rng.randrange(300, 900), rng.randrange(1200, 2500)])
        new = rng.randrange(6, 22)
        sc = SamplingConfig("random", temperature=0.8, seed=rng.randrange(1 << 20)) if i % 4 == 1 else SamplingConfig()
        reqs.append(dict(prompt_ids=random_tokens(plen, V, 4000 + 17 * seed + i), sampling=sc, max_new_tokens=new,
                         ignore_eos=True, request_id=i))
        need += -(-(plen + new) // ps)
    biggest = max(-(-(len(r["prompt_ids"]) + r["max_new_tokens"]) // ps) for r in reqs)
    opt = EngineOptions(dtype="bfloat16", page_size=ps, num_pages=max(biggest + 2, int(0.35 * need)), max_num_seqs=8,
                        max_num_batched_tokens=512, prefill_chunk=384, max_model_len=2600, use_graphs=True, run_ahead=True)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True
    arrivals = {}
    for r in reqs:
        arrivals.setdefault(rng.randrange(0, 10), []).append(r)
    drive(eng, arrivals)
    st = eng.scheduler.stats
    variants = sorted({v for g in eng.runner._graphs.values() for v in g._variants})
    print(f"seed {seed}: {st.steps} steps, {st.preemptions} preemptions, {eng.steps_ahead} launched ahead, "
          f"graphs {sorted(eng.runner._graphs)}, variants {variants}")
    assert True in seen["merge"], "no step cut a request's keys into several runs"
    for r in reqs:
        res = eng.pop_result(r["request_id"])
        assert res.finish_reason == "length" and len(res.output) == r["max_new_tokens"]
        check_choices(d, res, "bfloat16", r["sampling"])
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
