"""Replays the same requests whole, with the tail token by token, in portions
of changing size and mixed with other requests on a small pool, in 32-bit and
in bfloat16, and compares every position with the plain implementation."""
import pytest
import torch

import replay_lib as rl
from helpers import PAGE_SIZE, TOL, random_tokens, read_config

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = {"A": [1, 9, 40, 100], "B": [3, 17, 31, 64, 100, 150]}


def requests_for(name, model_dir):
    V = read_config(model_dir)["vocab_size"]
    return {f"{name}{i}": random_tokens(n, V, 1000 + 7 * i + n) for i, n in enumerate(LENGTHS[name])}


def make_runner(model_dir, dtype, page_size, num_pages, max_seqs=8):
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model = load_model(model_dir, DTYPES[dtype], "cuda:0")
    return ModelRunner(model, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("mode", ["whole", "tail", "chunks", "mixed"])
def test_replay_modes(model_dirs, name, dtype, mode):
    model_dir = model_dirs[name]
    reqs = requests_for(name, model_dir)
    steps = {"whole": rl.trace_whole, "tail": rl.trace_tail, "chunks": rl.trace_chunks,
             "mixed": rl.trace_mixed}[mode](reqs)
    ps = PAGE_SIZE[name]
    # the pool holds what is live at the worst moment and no more, so pages are used again
    num_pages = rl.max_live_tokens(steps, unit=ps) // ps
    runner = make_runner(model_dir, dtype, ps, num_pages)
    results = rl.run_steps_in_process(runner, steps)
    worst = rl.check_against_oracle(model_dir, reqs, steps, results, TOL[dtype])
    print(f"{name} {dtype} {mode}: worst rel. error {worst:.3e} over {len(steps)} steps, {num_pages} pages")
    assert all(g.pool.num_used == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, tmp_path, dtype):
    """The program itself, as a user calls it: mixed trace, files and 'done' lines."""
    model_dir = model_dirs["B"]
    reqs = requests_for("B", model_dir)
    steps = rl.trace_mixed(reqs, want_all=False)
    # some steps want nothing: no file may appear for them
    assert any(not any(e["want"] for e in s["entries"]) for s in steps)
    out = rl.run_steps_subprocess(model_dir, dtype, steps, str(tmp_path / "out"),
                                  rl.max_live_tokens(steps, 64))
    rl.check_against_oracle(model_dir, reqs, steps, out, TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("mode", ["tail", "mixed"])
def test_replay_with_decode_graphs(model_dirs, name, dtype, mode):
    """Decode-only steps run as replays of a captured HIP graph: every replay,
    with the engine's own eager steps between them, must match the plain
    implementation (a graph that bakes in a size or a table goes wrong on the
    second replay, not on the first)."""
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model_dir = model_dirs[name]
    reqs = requests_for(name, model_dir)
    steps = {"tail": rl.trace_tail, "mixed": rl.trace_mixed}[mode](reqs)
    ps = PAGE_SIZE[name]
    num_pages = rl.max_live_tokens(steps, unit=ps) // ps
    model = load_model(model_dir, DTYPES[dtype], "cuda:0")
    runner = ModelRunner(model, page_size=ps, num_pages=num_pages, max_seqs=4, use_graphs=True)
    results = rl.run_steps_in_process(runner, steps)
    assert runner._graphs, "no decode step went through a graph"
    decode_only = sum(1 for s in steps if s["entries"] and all(len(e["tokens"]) == 1 for e in s["entries"]))
    assert decode_only >= 3
    rl.check_against_oracle(model_dir, reqs, steps, results, TOL[dtype])
