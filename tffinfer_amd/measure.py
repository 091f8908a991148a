"""Measuring the engine: decode steps, prefill, a mixed workload, and what the
machine gives to kernels that do nothing else.

The reference's only timing is a wall clock around its decode loop that prints
tokens per second (src/core/runtime/InferRuntime.cu:347, :377-378).  Here a
phase is timed twice: by the wall clock around the whole phase, bracketed by
device synchronisations (what a caller sees, host work included), and by
device events between the steps, of which the median is reported (what the
device needs for a step, without the odd slow one).  ``bench.py`` at the
repository root and ``tffinfer --bench`` both call these functions.
"""
from __future__ import annotations

import math
import statistics
import time

import torch

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense, published


def _matrix_elements(part) -> int:
    """Elements of the matrices a part and its sub-parts multiply with."""
    n = sum(math.prod(spec.shape) for spec in part.weight_specs().values()
            if spec.init == "matrix" and len(spec.shape) == 2)
    return n + sum(_matrix_elements(child) for child in part.children().values())


def matrix_elements_per_step(model) -> int:
    """Elements of all matrices a step multiplies a token's row with, a layer that the run order
    names twice counted twice; without the output head."""
    return sum(_matrix_elements(model.blocks[call.layer]) for call in model.schedule)


def prefill_flops(model, T: int) -> float:
    """Flops of one prompt of T tokens, from the model's own parts: the matrix products of every
    layer call, what every mixer spends per (query, key) pair under its causal mask and window,
    and the output head for one row."""
    cfg = model.config
    flops = 2.0 * T * matrix_elements_per_step(model)
    for call in model.schedule:
        mixer = model.blocks[call.layer].mixer
        per_pair = mixer.flops_per_query_key_pair()
        if per_pair:
            spec = mixer.cache_spec()
            w = spec.window if spec is not None and spec.window > 0 else T
            w = min(w, T)
            pairs = w * (w + 1) / 2 + (T - w) * w      # token t reads min(t + 1, window) keys
            flops += per_pair * pairs
    return flops + 2.0 * cfg.hidden_size * cfg.vocab_size


def decode_bytes(model, batch: int, context: float, esz: int = 2) -> float:
    """Bytes a decode step has to read, from the model's own parts: every matrix it multiplies
    with once (a layer that the run order names twice, twice), the output head, and the keys and
    values that every layer call reads for the live requests (a window's worth where it has one)."""
    cfg = model.config
    weights = (matrix_elements_per_step(model) + cfg.hidden_size * cfg.vocab_size) * esz
    kv = 0.0
    for call in model.schedule:
        spec = model.blocks[call.layer].mixer.cache_spec()
        if spec is not None:
            keys = min(context, spec.window) if spec.window > 0 else context
            kv += 2 * spec.num_kv_heads * spec.head_dim * esz * batch * keys
    return weights + kv


def random_prompt(gen, n: int, vocab: int) -> list:
    return torch.randint(0, vocab, (n,), generator=gen).tolist()


def decode_slack(batch: int, context: int, chunk: int = 2048) -> int:
    """Steps the first request may decode while the last one still reads its prompt."""
    return batch * (-(-context // chunk) + 1)


def measure_prefill(engine, gen, T: int, vocab: int, reps: int = 5, warm: int = 2) -> dict:
    """One prompt of T tokens through the step function, ``reps`` times after ``warm`` untimed
    runs.  Returns the medians of the wall-clock times and of the device-event times, seconds."""
    from .engine.batch import StepEntry
    wall, dev = [], []
    for i in range(reps + warm):
        rid = f"prefill{i}"
        toks = random_prompt(gen, T, vocab)
        engine.runner.add_request(rid)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        logits = engine.runner.step([StepEntry(rid, toks, [T - 1])])
        e1.record()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert logits.shape[0] == 1
        engine.runner.free_request(rid)
        if i >= warm:   # the first runs warm up (allocator, work tables, clocks)
            wall.append(dt)
            dev.append(e0.elapsed_time(e1) / 1e3)
    return {"wall_s": statistics.median(wall), "device_s": statistics.median(dev), "reps": reps}


def measure_decode(engine, gen, batch: int, context, steps: int, warmup: int, vocab: int,
                   sampling=None) -> dict:
    """Fills ``batch`` requests with ``context`` tokens each (a list: request i with context[i];
    untimed prefill), then times
    ``steps`` decode steps of the whole engine (plan, tables, model, sampling, tokens back on
    the host).  ``wall_s``: all the steps by the wall clock between two synchronisations;
    ``step_median_s``: the median of the device-event intervals between consecutive steps.
    ``sampling``: a SamplingConfig for every request (its seed is offset by the request's number);
    greedy without one."""
    import dataclasses
    contexts = list(context) if isinstance(context, (list, tuple)) else [context] * batch
    for i in range(batch):
        # requests that finish their prompt early decode while the others still prefill
        engine.add_request(random_prompt(gen, contexts[i], vocab),
                           sampling=dataclasses.replace(sampling, seed=sampling.seed + i) if sampling else None,
                           max_new_tokens=warmup + steps + decode_slack(batch, max(contexts)) + 8, ignore_eos=True)
    # untimed: prompts, up to the first decode-only step
    while any(r.num_pending > 1 for r in engine.scheduler.running) or engine.scheduler.waiting:
        engine.step()
    for _ in range(warmup):
        out = engine.step()
        assert len(out) == batch
    events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    events[0].record()
    for i in range(steps):
        out = engine.step()
        events[i + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert len(out) == batch
    for r in list(engine.scheduler.running):
        engine.abort(r.id)
    while engine.has_work:      # a step launched ahead of the abort
        engine.step()
    gaps = [events[i].elapsed_time(events[i + 1]) / 1e3 for i in range(steps)]
    return {"wall_s": dt, "step_median_s": statistics.median(gaps), "step_min_s": min(gaps),
            "step_max_s": max(gaps), "steps": steps}


def measure_mixed(engine, gen, requests: int, vocab: int, new_tokens: int = 256, lo: int = 128,
                  hi: int = 4096) -> dict:
    """Continuous batching: all requests arrive at once, the scheduler admits them as
    slots and pages allow, cuts prompts into portions and decodes the others beside them."""
    engine.warm_up()      # (a server's start-up, not its work: the decode graphs of all batch sizes)
    lens = torch.randint(lo, hi + 1, (requests,), generator=gen).tolist()
    for n in lens:
        engine.add_request(random_prompt(gen, n, vocab), max_new_tokens=new_tokens, ignore_eos=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps = 0
    while engine.has_work:
        engine.step()
        steps += 1
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st = engine.scheduler.stats
    return {"requests": requests, "prompt_tokens": sum(lens), "generated_tokens": requests * new_tokens,
            "seconds": round(dt, 3), "engine_steps": steps, "preemptions": st.preemptions,
            "total_tokens_per_s": round((sum(lens) + requests * new_tokens) / dt, 1),
            "generated_tokens_per_s": round(requests * new_tokens / dt, 1)}


def quick_ceilings(device="cuda:0") -> dict:
    """The two ceilings the benchmark line prices its fractions against besides the published
    peaks, measured in the same process: streaming reads (GB/s) and back-to-back bfloat16
    MFMAs from registers (TFLOP/s)."""
    from .kernels import ops
    c = ops.measure_ceilings(device, gib=2.0, quick=True)
    return {"stream_read_GBps": c["stream_read_GBps"], "mfma_bf16_TFLOPs": c["mfma_bf16_TFLOPs_4_waves_per_simd"]}


def square_product_rates(device="cuda:0", n: int = 8192, reps: int = 5) -> dict:
    """A large square bfloat16 product [n, n] x [n, n]: the engine's own tiled kernel and, as a
    yardstick only (it is not on the engine's path), the vendor library's through torch."""
    from .kernels import ops
    dev = torch.device(device)
    a = torch.randn(n, n, dtype=torch.bfloat16, device=dev)
    w = torch.randn(n, n, dtype=torch.bfloat16, device=dev)
    wp = ops.pack_weight(w)

    def timed(fn):
        for _ in range(2):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize(dev)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize(dev)
        return e0.elapsed_time(e1) / 1e3 / reps

    flops = 2.0 * n * n * n
    ours = timed(lambda: ops.linear(a, wp))
    lib = timed(lambda: torch.matmul(a, w.t()))
    return {"square_product_n": n, "square_product_TFLOPs": round(flops / ours / 1e12, 1),
            "square_product_library_TFLOPs": round(flops / lib / 1e12, 1)}
