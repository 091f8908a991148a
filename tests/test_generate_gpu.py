"""Generation through the entry points against the plain implementation."""
import json
import os
import subprocess
import sys

import pytest
import torch

from helpers import note_error, tol, oracle_logits, random_tokens, read_config, rel_err
from plain_qwen3 import plain_greedy, plain_inverse_cdf, plain_probs

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_generate_greedy(model_dir, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(plain_greedy(oracle_logits(model_dir, toks)[-1]))
    return toks[len(prompt):]


def check_choices(model_dir, result, dtype, sampling=None):
    """Every kept logits row matches the plain logits of the engine's own
    sequence at that place, and the chosen token is what the plain sampler
    picks from that row."""
    from tffinfer_amd.sampling import uniform_at
    seq = result.prompt + result.output
    ref = oracle_logits(model_dir, seq)
    assert len(result.logits) == len(result.output)
    for i, (row, tok) in enumerate(zip(result.logits, result.output)):
        pos = len(result.prompt) + i - 1
        err = rel_err(row, ref[pos])
        note_error(dtype, model_dir, err)
        assert err <= tol(dtype, model_dir), f"output {i}: {err:.3e}"
        if sampling is None or sampling.greedy:
            assert tok == plain_greedy(row)
        else:
            t, k, p, m = sampling.effective()
            assert tok == plain_inverse_cdf(plain_probs(row, t, k, p, m), uniform_at(sampling.seed, i))


def test_greedy_through_the_reference_style_entry_point_fp32(model_dirs):
    from tffinfer_amd import LLMInferRuntime, ModelConfig
    d = model_dirs["A"]
    V = read_config(d)["vocab_size"]
    prompts = [random_tokens(n, V, 50 + n) for n in (1, 9, 40)]
    cfg = ModelConfig()
    cfg._use_f16 = False
    cfg._n_ctx = 128
    rt = LLMInferRuntime()
    assert rt.load_model([d], cfg) and rt.init_runtime_context()
    assert rt.encode(prompts) == 50
    out = []
    assert rt.infer(16, out)
    assert out == [plain_generate_greedy(d, p, 16) for p in prompts]


@pytest.mark.parametrize("name", ["A", "C"])    # (C: the head size of the large models and its decode kernels)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_engine(model_dirs, dtype, name):
    from tffinfer_amd import EngineOptions, LLMEngine
    d = model_dirs[name]
    V = read_config(d)["vocab_size"]
    prompts = [random_tokens(n, V, 60 + n) for n in (1, 9, 40)]
    eng = LLMEngine.from_model_dir(d, EngineOptions(dtype=dtype, page_size=16, kv_tokens=256, max_num_seqs=4))
    eng.keep_logits = True
    res = eng.generate(prompts, max_new_tokens=16, ignore_eos=True)
    for r in res:
        assert len(r.output) == 16 and r.finish_reason == "length"
        check_choices(d, r, dtype)


@pytest.mark.parametrize("name", ["B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_chunked_prefill_mixed_with_decode_temperature_small_pool(model_dirs, dtype, name):
    """Tiny B's workload (and with C's head size): 5 requests, portions of 24 tokens beside
    decoding, 24 tokens at temperature 0.8 with a fixed seed, on a pool so small that
    requests are preempted and computed again."""
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    d = model_dirs[name]
    V = read_config(d)["vocab_size"]
    prompts = [random_tokens(n, V, 70 + n) for n in (3, 17, 31, 64, 100)]
    sc = [SamplingConfig("random", temperature=0.8, seed=100 + i) for i in range(5)]
    opt = EngineOptions(dtype=dtype, page_size=8, num_pages=20, max_num_seqs=4, max_num_batched_tokens=48,
                        prefill_chunk=24)
    eng = LLMEngine.from_model_dir(d, opt)
    eng.keep_logits = True
    res = eng.generate(prompts, sc, max_new_tokens=24, ignore_eos=True)
    assert eng.scheduler.stats.preemptions > 0, "the pool was meant to run out"
    for r, s in zip(res, sc):
        assert len(r.output) == 24
        # logits kept before a preemption stay valid: the recomputation feeds the same tokens
        r.logits = r.logits[:len(r.output)]
        check_choices(d, r, dtype, s)
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
    if dtype == "float32":
        # each request alone gives the same tokens as in the crowd
        for p, s, r in zip(prompts, sc, res):
            alone = LLMEngine(eng.model, EngineOptions(dtype=dtype, page_size=8, num_pages=40, max_num_seqs=1))
            assert alone.generate([p], s, max_new_tokens=24, ignore_eos=True)[0].output == r.output


def test_sampling_filters_and_penalty_through_engine(model_dirs):
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    d = model_dirs["A"]
    prompts = [[5, 6, 7, 8], [9, 10]]
    sc = [SamplingConfig("top_k", 0.9, top_k=7, top_p=0.9, seed=4), SamplingConfig("top_p", 1.2, top_p=0.6, min_p=0.01, seed=5)]
    eng = LLMEngine.from_model_dir(d, EngineOptions(dtype="float32", kv_tokens=128, max_num_seqs=2))
    eng.keep_logits = True
    res = eng.generate(prompts, sc, max_new_tokens=12, ignore_eos=True)
    for r, s in zip(res, sc):
        check_choices(d, r, "float32", s)
    # repetition penalty: the kept rows are the logits before the penalty
    from plain_qwen3 import plain_repetition_penalty
    r = eng.generate([[1, 2, 3]], SamplingConfig("greedy", repetition_penalty=5.0), max_new_tokens=20,
                     ignore_eos=True)[0]
    for i, (row, tok) in enumerate(zip(r.logits, r.output)):
        seen = r.prompt + r.output[:i]
        assert tok == plain_greedy(plain_repetition_penalty(row, seen, 5.0))
    plain = eng.generate([[1, 2, 3]], SamplingConfig("greedy"), max_new_tokens=20, ignore_eos=True)[0].output
    assert plain != r.output, "a penalty of 5 was expected to change a tiny model's greedy loop"


def test_sampler_parameters_go_round_the_pinned_ring():
    """The sampler sends its per-row parameters through a ring of pinned buffers, one copy a
    call: more calls in a row than the ring has buffers, batches of changing size (one of them
    beyond a buffer's first size), penalties beside draws, every token against the plain
    implementation."""
    from tffinfer_amd.sampling import Sampler, SamplingConfig, uniform_at
    from plain_qwen3 import plain_repetition_penalty
    sampler = Sampler(torch.device("cuda:0"))
    V = 300
    g = torch.Generator().manual_seed(9)
    for call, R in enumerate([3, 1, 7, 1500, 2, 5, 4, 6, 1, 3]):
        logits = torch.randn(R, V, generator=g) * 2
        configs = [SamplingConfig(type=["top_k", "top_p", "random", "greedy"][(r + call) % 4], temperature=0.5 + 0.1 * (r % 7),
                                  top_k=[0, 5, 40][r % 3], top_p=[1.0, 0.9, 0.6][(r + call) % 3], min_p=[0.0, 0.02][r % 2],
                                  repetition_penalty=1.0 if (r + call) % 5 else 1.3, seed=100 * call + r) for r in range(R)]
        indices = [(7 * r + call) % 50 for r in range(R)]
        seen = [[(r * 13 + j) % V for j in range(1 + r % 9)] for r in range(R)]
        got = sampler.sample(logits.to("cuda:0"), configs, indices, seen)
        for r in range(0, R, max(1, R // 12)):
            c = configs[r]
            x = plain_repetition_penalty(logits[r], seen[r], c.repetition_penalty) if c.repetition_penalty != 1.0 else logits[r]
            if c.greedy:
                assert got[r] == plain_greedy(x), (call, r)
            else:
                ref = plain_probs(x, c.temperature, c.top_k, c.top_p, c.min_p)
                assert got[r] == plain_inverse_cdf(ref, uniform_at(c.seed, indices[r])), (call, r)


def test_eos_stops(model_dirs):
    from tffinfer_amd import EngineOptions, LLMEngine
    d = model_dirs["A"]
    eng = LLMEngine.from_model_dir(d, EngineOptions(dtype="float32", kv_tokens=128, max_num_seqs=2))
    full = eng.generate([[3, 4, 5]], max_new_tokens=10, ignore_eos=True)[0].output
    stop = eng.generate([[3, 4, 5]], max_new_tokens=10, eos_token_id=full[4])[0]
    cut = full.index(full[4]) + 1
    assert stop.output == full[:cut] and stop.finish_reason == "stop"


@pytest.mark.parametrize("dtype,use_graphs", [("float32", True), ("bfloat16", True), ("bfloat16", False)])
def test_steps_launched_ahead_give_the_same_tokens(model_dirs, dtype, use_graphs):
    """Decode steps launched before the tokens of the step in flight are read: the same
    outputs as with one step at a time, with requests that end at different lengths, one
    that ends on a token of its own choosing, more requests than slots and a pool that
    runs out.  (A request that ends is noticed a step later when steps are launched ahead, so
    the next one is admitted a step later and some tokens are computed in other batches, by
    other kernels, than with one step at a time: equal to rounding, which with this model and
    these seeds flips no choice.  What the engine computes is checked against the plain
    implementation, with tolerances, by the tests above.)"""
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    d = model_dirs["B"]
    V = read_config(d)["vocab_size"]
    prompts = [random_tokens(n, V, 170 + n) for n in (3, 17, 31, 9, 26, 5)]
    sc = [SamplingConfig("random", temperature=0.7, seed=30 + i) if i % 2 else SamplingConfig() for i in range(6)]
    lens = [24, 7, 30, 16, 1, 21]
    outs = {}
    for ahead in (False, True):
        opt = EngineOptions(dtype=dtype, page_size=8, num_pages=24, max_num_seqs=4, max_num_batched_tokens=48,
                            prefill_chunk=24, run_ahead=ahead, use_graphs=use_graphs)
        eng = LLMEngine.from_model_dir(d, opt)
        eos = None
        if ahead:   # request 2 stops at the token it chose as its 12th
            eos = outs[False][2][11]
        for i, (p, s, n) in enumerate(zip(prompts, sc, lens)):
            eng.add_request(p, s, max_new_tokens=n, ignore_eos=not (eos is not None and i == 2),
                            eos_token_id=eos if i == 2 else None, request_id=i)
        got = {i: [] for i in range(6)}
        fin = {}
        while eng.has_work:
            for rid, tok, done in eng.step():
                got[rid].append(tok)
                if done:
                    fin[rid] = True
        assert len(fin) == 6
        assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
        assert (eng.steps_ahead > 10) == ahead
        outs[ahead] = got
    for i in range(6):
        want = outs[False][i]
        if i == 2:
            want = want[:want.index(want[11]) + 1]
        assert outs[True][i] == want, f"request {i}"
        assert len(outs[False][i]) == lens[i]


def test_command_line(model_dirs):
    d = model_dirs["A"]
    prompt = [7, 8, 9, 10, 11]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "tffinfer"), d, "--fp32", "--prompt-ids",
           ",".join(map(str, prompt)), "--n-predict", "8", "--n-ctx", "128", "--json", "--ignore-eos"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr
    rec = json.loads(p.stdout.strip().splitlines()[-1])
    assert rec["prompt"] == prompt and rec["output"] == plain_generate_greedy(d, prompt, 8)
    p = subprocess.run([sys.executable, "-m", "tffinfer_amd", d, "--load-only"], capture_output=True, text=True,
                       timeout=300, cwd=ROOT)
    assert p.returncode == 0 and "loaded" in p.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_warm_up_captures_every_decode_graph_beforehand(model_dirs, dtype):
    """An engine that was warmed up has the graph of every batch size and captures none while it
    works; its tokens are those of an engine that captures as it goes.  The latter lets a larger
    graph stand in for a half-way bucket that is wanted only in passing."""
    from tffinfer_amd import EngineOptions, LLMEngine
    d = model_dirs["A"]
    V = read_config(d)["vocab_size"]
    prompts = [random_tokens(n, V, 400 + n) for n in (5, 9, 4, 12, 7, 3)]
    lens = [20, 6, 14, 9, 17, 11]
    outs = []
    for warm in (False, True):
        eng = LLMEngine.from_model_dir(d, EngineOptions(dtype=dtype, page_size=8, kv_tokens=512, max_num_seqs=6))
        assert eng.runner._graph_buckets == [1, 2, 3, 4, 6]
        if warm:
            assert eng.warm_up() == 5 and eng.warm_up() == 0
        for i, (p, n) in enumerate(zip(prompts, lens)):
            eng.add_request(p, max_new_tokens=n, ignore_eos=True, request_id=i)
        while eng.has_work:
            eng.step()
        outs.append([eng.pop_result(i).output for i in range(6)])
        captured = sorted(eng.runner._graphs)
        if warm:
            assert captured == [1, 2, 3, 4, 6]
        else:
            assert captured == [1, 3, 6]      # 6 stood in for 4 and 3 for 2, which were wanted for a few steps only
    assert outs[0] == outs[1]


@pytest.mark.parametrize("name", ["B", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_groups_get_pools_of_their_own_size(model_dirs, dtype, name):
    """Sized by the engine (not by a page count given to it), the layers with a window get the
    pages their window and a step's tokens need, a fraction of the pool of the layers that keep
    every key; requests far longer than that pool run beside each other without a preemption."""
    from tffinfer_amd import EngineOptions, LLMEngine, SamplingConfig
    from tffinfer_amd.cache.sizing import window_pool_pages
    d = model_dirs[name]
    cfg = read_config(d)
    V, limit = cfg["vocab_size"], cfg["max_position_embeddings"]
    opt = EngineOptions(dtype=dtype, page_size=8, max_num_seqs=4, max_num_batched_tokens=64, prefill_chunk=24)
    eng = LLMEngine.from_model_dir(d, opt)
    groups = {g.spec.window: g.pool.num_pages for g in eng.runner.cache.groups}
    w = cfg["sliding_window"]
    assert groups[0] == 4 * limit // 8 + 4
    assert groups[w] == window_pool_pages(w, 8, 4, 64) < groups[0] // 3
    prompts = [random_tokens(n, V, 80 + n) for n in (limit - 60, 150, 9, 120, 77)]
    sc = [SamplingConfig("random", temperature=0.8, seed=7 + i) if i % 2 else SamplingConfig() for i in range(5)]
    eng.keep_logits = True
    res = eng.generate(prompts, sc, max_new_tokens=40, ignore_eos=True)
    assert eng.scheduler.stats.preemptions == 0
    for r, s in zip(res, sc):
        assert len(r.output) == 40
        check_choices(d, r, dtype, s)
    assert all(g.pool.num_used == 0 for g in eng.runner.cache.groups)
