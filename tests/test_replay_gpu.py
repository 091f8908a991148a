"""Replays the same requests whole, with the tail token by token, in portions
of changing size and mixed with other requests on a small pool, in 32-bit and
in bfloat16, and compares every position with the plain implementation."""
import pytest
import torch

import replay_lib as rl
from helpers import PAGE_SIZE, tol, random_tokens, read_config, rel_err

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = {"A": [1, 9, 40, 100], "B": [3, 17, 31, 64, 100, 150], "C": [2, 33, 70, 129, 200], "D": [5, 41, 90, 160],
           "B0": [3, 17, 31, 64, 100, 150]}


def requests_for(name, model_dir):
    V = read_config(model_dir)["vocab_size"]
    return {f"{name}{i}": random_tokens(n, V, 1000 + 7 * i + n) for i, n in enumerate(LENGTHS[name])}


def make_runner(model_dir, dtype, page_size, num_pages, max_seqs=8):
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model = load_model(model_dir, DTYPES[dtype], "cuda:0")
    return ModelRunner(model, page_size=page_size, num_pages=num_pages, max_seqs=max_seqs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "B0"])
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
    worst = rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype)
    print(f"{name} {dtype} {mode}: worst rel. error {worst:.3e} over {len(steps)} steps, {num_pages} pages")
    assert all(g.pool.num_used == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,ps", [("B", 24), ("C", 40)])
def test_replay_with_pages_that_are_no_power_of_two(model_dirs, name, ps, dtype):
    """The matrix-core attention takes pages of a power of two of tokens; with other page sizes
    the bfloat16 engine runs the general attention kernel, and nothing else changes."""
    from tffinfer_amd.kernels import ops
    assert not ops.mfma_attention_supported(torch.bfloat16, 128, ps)
    model_dir = model_dirs[name]
    reqs = requests_for(name, model_dir)
    steps = rl.trace_mixed(reqs)
    runner = make_runner(model_dir, dtype, ps, rl.max_live_tokens(steps, unit=ps) // ps)
    results = rl.run_steps_in_process(runner, steps)
    rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype)


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
    rl.check_against_oracle(model_dir, reqs, steps, out, tol(dtype, "B"), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "B0"])
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
    rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "B0"])     # (C's and D's head sizes take the decode kernel that writes keys itself)
def test_padding_rows_of_a_graph_write_nothing(model_dirs, name, dtype):
    """Three requests decode through the graph of four rows: the fourth row is padding (token 0
    at position 0 with a block table of zeros).  After every step the caches must hold, bit for
    bit, what the same steps leave without graphs: nothing of the padding row may reach page 0
    or any other page."""
    from tffinfer_amd.engine.batch import StepEntry
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model_dir = model_dirs[name]
    V = read_config(model_dir)["vocab_size"]
    ps = PAGE_SIZE[name]
    prompts = {f"r{i}": random_tokens(5 + 7 * i, V, 300 + i) for i in range(3)}
    runners = [ModelRunner(load_model(model_dir, DTYPES[dtype], "cuda:0"), page_size=ps, num_pages=24, max_seqs=4,
                           use_graphs=g) for g in (False, True)]
    for rn in runners:
        for rid, toks in prompts.items():
            rn.add_request(rid)
        rn.step([StepEntry(rid, toks, []) for rid, toks in prompts.items()])
    for step in range(6):
        toks = {rid: (step * 13 + i * 5 + 1) % V for i, rid in enumerate(prompts)}
        logits = [rn.step([StepEntry(rid, [toks[rid]], [0]) for rid in prompts]).clone() for rn in runners]
        assert torch.equal(logits[0], logits[1]), f"logits differ at decode step {step}"
        for (k0, v0), (k1, v1) in zip(_all_caches(runners[0]), _all_caches(runners[1])):
            assert torch.equal(k0, k1) and torch.equal(v0, v1), f"caches differ after decode step {step}"
    assert runners[1]._graphs and not runners[0]._graphs


def _all_caches(runner):
    out, seen = [], set()
    for cache_id, _, kvspec, _ in runner.model.call_requirements():
        if kvspec is not None and cache_id not in seen:
            seen.add(cache_id)
            out.append(runner.cache.kv_tensors(cache_id))
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n", [("A", 128), ("B", 256), ("C", 300), ("D", 320), ("B0", 256)])
@pytest.mark.parametrize("graphs", [False, True])
def test_long_decoding(model_dirs, name, dtype, n, graphs):
    """A few prompt tokens, then one token a step up to the model's longest
    position: every position against the plain implementation (B's window
    passes its pages many times over)."""
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    model_dir = model_dirs[name]
    V = read_config(model_dir)["vocab_size"]
    reqs = {"long": random_tokens(n, V, 4242)}
    steps = rl.trace_tail(reqs, tail=n - 5)
    ps = PAGE_SIZE[name]
    runner = ModelRunner(load_model(model_dir, DTYPES[dtype], "cuda:0"), page_size=ps,
                         num_pages=-(-n // ps), max_seqs=2, use_graphs=graphs)
    results = rl.run_steps_in_process(runner, steps)
    rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype)
    if name in ("B", "D"):   # the window groups gave pages back on the way
        assert any(g.spec.window > 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "B0"])
def test_first_tokens(model_dirs, name, dtype):
    """Sequences of one, two and three tokens: whole, and token by token."""
    model_dir = model_dirs[name]
    V = read_config(model_dir)["vocab_size"]
    reqs = {f"s{n}": random_tokens(n, V, 90 + n) for n in (1, 2, 3)}
    for steps in (rl.trace_whole(reqs), rl.trace_tail(reqs, tail=3)):
        runner = make_runner(model_dir, dtype, PAGE_SIZE[name], 4)
        results = rl.run_steps_in_process(runner, steps)
        rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, name), dtype)


MID = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=1024, num_hidden_layers=3,
    num_attention_heads=16, num_key_value_heads=4, head_dim=64, intermediate_size=8200,
    vocab_size=9000, max_position_embeddings=2048, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=True,
)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_midsize_model_long_prompt(tmp_path_factory, dtype):
    """Sizes at which the large-tile products, the gated epilogue and the
    two-tile attention kernel run: a prompt of 1,100 tokens whole, in portions
    of 512, and followed by decoding, against the plain implementation."""
    from helpers import make_model_dir
    model_dir = make_model_dir(str(tmp_path_factory.mktemp("mid") / "m"), MID, 5)
    toks = random_tokens(1100, MID["vocab_size"], 77)
    reqs = {"p": toks}
    look = [0, 1, 63, 64, 500, 1023, 1024, 1087]
    whole = [{"step": 0, "entries": [{"id": "p", "tokens": toks[:1088], "want": look}], "end": []}]
    whole += [{"step": 1 + i, "entries": [{"id": "p", "tokens": [toks[1088 + i]], "want": [0]}],
               "end": ["p"] if i == 11 else []} for i in range(12)]
    parts, done = [], 0
    for n in (512, 512, 64, 12):
        want = [w - done for w in look if done <= w < done + n]
        parts.append({"step": len(parts), "entries": [{"id": "p", "tokens": toks[done:done + n], "want": want}],
                      "end": ["p"] if done + n == 1100 else []})
        done += n
    for steps in (whole, parts):
        runner = make_runner(model_dir, dtype, 16, 72, max_seqs=2)
        results = rl.run_steps_in_process(runner, steps)
        worst = rl.check_against_oracle(model_dir, reqs, steps, results, tol(dtype, "mid"), dtype)
        print(f"mid {dtype}: worst rel. error {worst:.3e}")


LARGE_SHAPES = {
    # the layer sizes of larger members of the family, one layer each
    "14b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, head_dim=128, intermediate_size=17408),
    "32b": dict(hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128, intermediate_size=25600),
}


@pytest.mark.parametrize("shape", ["14b", "32b"])
def test_large_layer_sizes_against_the_plain_implementation(shape, tmp_path):
    """One layer with the widths of the 14B and 32B models (inner sizes that are no power of
    two, 5 and 8 query heads to a key head), weights from a folder: the float32 engine and the
    bfloat16 engine against the plain implementation (in float64; its matrix products run on
    the GPU here, the widths being what they are), for a prompt in portions beside another
    request, then steps of two decoding requests.  The kernels that only these widths reach
    (tiles that split K, the streaming product's other shapes) are thus pinned to the plain
    implementation directly, not only to the engine's other precision."""
    from plain_qwen3 import fast_forward, load_plain_model
    from tffinfer_amd.engine.batch import StepEntry
    from tffinfer_amd.engine.runner import ModelRunner
    from tffinfer_amd.models import load_model
    from tffinfer_amd.weights import write_random_model
    cfg = dict(architectures=["Qwen3ForCausalLM"], num_hidden_layers=1, vocab_size=5003,
               max_position_embeddings=2048, rms_norm_eps=1e-6, rope_theta=1000000.0,
               tie_word_embeddings=False, **LARGE_SHAPES[shape])
    V = cfg["vocab_size"]
    d = write_random_model(str(tmp_path / shape), cfg, seed=11)
    a, b = random_tokens(712, V, 5), random_tokens(47, V, 6)
    steps = [[("a", a[:512], [0, 100, 511])], [("a", a[512:700], [187]), ("b", b[:40], [39])]]
    steps += [[("a", [a[700 + i]], [0]), ("b", [b[40 + i]], [0])] for i in range(7)]
    steps += [[("a", a[707:712], [0, 4])]]
    # the plain logits at the places the steps ask for, in their order
    pcfg, raw = load_plain_model(d, torch.float64)
    raw = {k: v.cuda() for k, v in raw.items()}
    full = {"a": fast_forward(pcfg, raw, a).cpu(), "b": fast_forward(pcfg, raw, b).cpu()}
    del raw
    torch.cuda.empty_cache()
    want, done = [], {"a": 0, "b": 0}
    for st in steps:
        for r, t, w in st:
            want += [full[r][done[r] + i] for i in w]
            done[r] += len(t)
    want = torch.stack(want)
    out = {}
    for dtype in (torch.float32, torch.bfloat16):
        model = load_model(d, dtype, "cuda:0")
        runner = ModelRunner(model, page_size=16, num_pages=64, max_seqs=2)
        runner.add_request("a")
        runner.add_request("b")
        rows = []
        for st in steps:
            rows.append(runner.step([StepEntry(r, list(t), list(w)) for r, t, w in st]).float().cpu())
        out[dtype] = torch.cat(rows)
        del runner, model
        torch.cuda.empty_cache()
    assert out[torch.float32].shape[0] == 3 + 2 + 14 + 2 == want.shape[0]
    e32, e16 = rel_err(out[torch.float32], want), rel_err(out[torch.bfloat16], want)
    print(f"{shape}: against the plain implementation, float32 {e32:.3e}, bfloat16 {e16:.3e}; "
          f"bfloat16 against float32 {rel_err(out[torch.bfloat16], out[torch.float32]):.3e}")
    assert e32 <= tol("float32", "large")
    assert e16 <= tol("bfloat16", "large")
