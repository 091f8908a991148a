"""Builds replay traces (the JSON steps bin/trace_run reads) and checks what a
replay returns against the plain implementation."""
from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np
import torch

from helpers import note_error, oracle_logits, rel_err

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHUNK_CYCLE = [7, 2, 13, 3, 2, 24, 5, 2, 16, 9]


def trace_whole(requests: dict) -> list[dict]:
    """Each request alone and whole, every position wanted."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [
            {"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def trace_tail(requests: dict, tail: int = 32) -> list[dict]:
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": list(toks[:head]), "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": [toks[i]], "want": [0]}], "end": [rid] if i == len(toks) - 1 else []})
    return steps


def trace_chunks(requests: dict, cycle=CHUNK_CYCLE) -> list[dict]:
    """Portions of changing size, down to two tokens."""
    steps = []
    c = 0
    for rid, toks in requests.items():
        i = 0
        while i < len(toks):
            n = min(cycle[c % len(cycle)], len(toks) - i)
            c += 1
            last = i + n == len(toks)
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": list(toks[i:i + n]), "want": list(range(n))}],
                "end": [rid] if last else []})
            i += n
    return steps


def trace_mixed(requests: dict, max_live: int = 4, prompt_frac: float = 0.6, cycle=CHUNK_CYCLE,
                want_all: bool = True) -> list[dict]:
    """Up to ``max_live`` requests at a time: the first ``prompt_frac`` of each
    request's tokens come in portions of changing size, the rest one token a
    step, so portions of some stand beside single tokens of others.  A request
    is sometimes left out of a step.  Finished requests end and the next one
    is admitted, so pages are used again."""
    waiting = list(requests.items())
    live = []   # [rid, toks, done, prompt_len]
    steps = []
    c = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live.append([rid, list(toks), 0, max(1, int(len(toks) * prompt_frac))])
        entries, ended = [], []
        for k, item in enumerate(live):
            rid, toks, done, plen = item
            if (len(steps) + k) % 5 == 4 and len(live) > 1:
                continue  # left out of this step, goes on later
            if done < plen:
                n = min(cycle[c % len(cycle)], plen - done)
                c += 1
            else:
                n = 1
            want = list(range(n)) if want_all else ([n - 1] if done + n == len(toks) else [])
            entries.append({"id": rid, "tokens": toks[done:done + n], "want": want})
            item[2] = done + n
            if item[2] == len(toks):
                ended.append(rid)
        live = [it for it in live if it[0] not in ended]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def max_live_tokens(steps, unit: int = 64) -> int:
    """Most tokens live requests hold at any time, each rounded up to ``unit``."""
    held, best = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        best = max(best, sum(-(-v // unit) * unit for v in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return best


def run_steps_in_process(runner, steps) -> dict:
    """Drives a ModelRunner as bin/trace_run does.  Returns {step: logits}."""
    from tffinfer_amd.engine.batch import StepEntry
    out = {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if not runner.has_request(e["id"]):
                runner.add_request(e["id"])
            entries.append(StepEntry(e["id"], list(e["tokens"]), list(e["want"])))
        logits = runner.step(entries)
        if logits.shape[0]:
            out[s["step"]] = logits.float().cpu()
        for rid in s["end"]:
            runner.free_request(rid)
        runner.cache.check()
    return out


def run_steps_subprocess(model_dir, dtype, steps, out_dir, max_tokens, extra_args=(), env=None) -> dict:
    """Runs bin/trace_run as a user would and reads back its files."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens), *extra_args]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for s in steps:
            p.stdin.write(json.dumps(s) + "\n")
            p.stdin.flush()
            line = p.stdout.readline().strip()
            assert line == f"done {s['step']}", f"expected 'done {s['step']}', got {line!r}"
        p.stdin.close()
        assert p.wait(timeout=120) == 0
    finally:
        if p.poll() is None:
            p.kill()
    with open(os.path.join(model_dir, "config.json")) as f:
        V = json.load(f)["vocab_size"]
    out = {}
    for s in steps:
        path = os.path.join(out_dir, f"{s['step']}.f32")
        n = sum(len(e["want"]) for e in s["entries"])
        if n:
            out[s["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n, V).copy())
        else:
            assert not os.path.exists(path)
    return out


def check_against_oracle(model_dir, requests, steps, results, tol, dtype: str | None = None) -> float:
    """Every wanted row must match the plain implementation's logits at that
    request's position.  Returns the largest relative error; on a failure names
    the first wrong token."""
    done = {rid: 0 for rid in requests}
    worst = 0.0
    for s in steps:
        row = 0
        for e in s["entries"]:
            rid = e["id"]
            ref = oracle_logits(model_dir, requests[rid])
            for w in e["want"]:
                pos = done[rid] + w
                got = results[s["step"]][row]
                err = rel_err(got, ref[pos])
                worst = max(worst, err)
                assert err <= tol, (
                    f"step {s['step']}: request {rid!r} position {pos} (token {w} of a portion of "
                    f"{len(e['tokens'])} starting at {done[rid]}): rel. error {err:.3e} > {tol:.1e}")
                row += 1
            done[rid] += len(e["tokens"])
        if s["step"] in results:
            assert row == results[s["step"]].shape[0]
    if dtype is not None:
        note_error(dtype, model_dir, worst)
    return worst
