"""The Python side of the C interface of the engine (csrc/tffinfer_engine.h).

The C library embeds the interpreter and calls the functions below with plain
values: strings (JSON for options and per-request parameters), ``bytes`` of
int32 token ids, integers.  They return integers or ``bytes`` that the C side
copies into the caller's buffers.  Nothing here computes anything: it is the
package's engine, scheduler, step function and cache that run.

The reference exports its runtime class to C++ callers through a visibility
macro (include/ExportInc.h:6-16, src/core/runtime/InferRuntime.h:32); the calls
here follow that class's life cycle (load_model, init_runtime_context, encode,
infer: src/core/runtime/InferRuntime.h:34-45) cut into requests and steps.
"""
from __future__ import annotations

import json
import struct

import numpy as np

_ENGINE_KEYS = ("dtype", "device", "page_size", "num_pages", "kv_tokens", "kv_bytes", "max_num_seqs",
                "max_num_batched_tokens", "prefill_chunk", "max_model_len", "memory_fraction", "use_graphs",
                "run_ahead", "warm_up", "token_quantum")
_SAMPLING_KEYS = ("type", "temperature", "top_k", "top_p", "min_p", "repetition_penalty", "seed")
_REQUEST_KEYS = ("max_new_tokens", "eos_token_id", "ignore_eos", "sampling")


def _options(options_json: str):
    from .engine import EngineOptions
    given = json.loads(options_json) if options_json else {}
    if not isinstance(given, dict):
        raise ValueError("options: a JSON object is expected")
    unknown = sorted(set(given) - set(_ENGINE_KEYS))
    if unknown:
        raise ValueError(f"options: unknown keys {unknown}; known: {list(_ENGINE_KEYS)}")
    return EngineOptions(**given)


class Handle:
    """An engine and what the C interface keeps beside it: events of a step that did not fit the
    caller's buffer, and the requests that raw steps have opened."""

    def __init__(self, engine):
        self.engine = engine
        self.events: list[tuple[int, int, int]] = []
        self.raw: set = set()


def create(model_dir: str, options_json: str) -> Handle:
    from .engine import LLMEngine
    return Handle(LLMEngine.from_model_dir(model_dir, _options(options_json)))


def create_random(config_file: str, seed: int, options_json: str) -> Handle:
    """An engine over seeded random weights and no files: the weights are those that the random
    mode of the weights module writes into a folder for the same configuration and seed."""
    import torch
    from .engine import LLMEngine
    from .engine.llm_engine import resolve_dtype
    from .models import build_model_skeleton, config_from_dict
    opt = _options(options_json)
    with open(config_file) as f:
        config = config_from_dict(json.load(f))
    dtype = resolve_dtype(opt.dtype)
    model = build_model_skeleton(config)
    model.init_random(int(seed), dtype, opt.device)
    return Handle(LLMEngine(model, opt))


def vocab_size(h: Handle) -> int:
    return int(h.engine.model.config.vocab_size)


def add_request(h: Handle, ids: bytes, params_json: str) -> int:
    from .sampling import SamplingConfig
    p = json.loads(params_json) if params_json else {}
    if not isinstance(p, dict):
        raise ValueError("request parameters: a JSON object is expected")
    unknown = sorted(set(p) - set(_REQUEST_KEYS))
    if unknown:
        raise ValueError(f"request parameters: unknown keys {unknown}; known: {list(_REQUEST_KEYS)}")
    s = p.get("sampling") or {}
    bad = sorted(set(s) - set(_SAMPLING_KEYS))
    if bad:
        raise ValueError(f"sampling: unknown keys {bad}; known: {list(_SAMPLING_KEYS)}")
    tokens = np.frombuffer(ids, dtype="<i4").tolist()
    if not tokens:
        raise ValueError("a request needs at least one token")
    rid = h.engine.add_request(tokens, SamplingConfig(**s), int(p.get("max_new_tokens", 64)),
                               p.get("eos_token_id"), bool(p.get("ignore_eos", False)))
    return int(rid)


def step(h: Handle, capacity: int) -> bytes:
    """Events (request id int64, token int32 or -1, finished int32), at most ``capacity`` of them.
    Events of an earlier step that did not fit come first, and no new step runs while there are any."""
    if not h.events:
        for rid, tok, fin in h.engine.step():
            h.events.append((int(rid), -1 if tok is None else int(tok), 1 if fin else 0))
            if fin:
                h.engine.pop_result(rid)        # the C caller has every token already
    out, h.events = h.events[:capacity], h.events[capacity:]
    return b"".join(struct.pack("<qii", *e) for e in out)


def has_work(h: Handle) -> int:
    return 1 if (h.events or h.engine.has_work) else 0


def abort(h: Handle, rid: int) -> int:
    return 1 if h.engine.abort(rid) else 0


def step_raw(h: Handle, ids: list, tokens: list, wants: list) -> bytes:
    """One call of the step function with the entries as given: no scheduler, no sampling.
    Returns the float32 logits [wanted, vocab] of the wanted places, entries in order."""
    import torch
    from .engine.batch import StepEntry
    runner = h.engine.runner
    entries = []
    for rid, tok, want in zip(ids, tokens, wants):
        key = ("raw", int(rid))
        if not runner.has_request(key):
            runner.add_request(key)
            h.raw.add(key)
        entries.append(StepEntry(key, np.frombuffer(tok, dtype="<i4").tolist(), np.frombuffer(want, dtype="<i4").tolist()))
    logits = runner.step(entries)
    if logits.shape[0] == 0:
        torch.cuda.synchronize()
        return b""
    return logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4", copy=False).tobytes()


def end_raw(h: Handle, rid: int) -> int:
    key = ("raw", int(rid))
    if key not in h.raw:
        return 0
    h.engine.runner.free_request(key)
    h.raw.discard(key)
    return 1


def destroy(h: Handle) -> None:
    for key in list(h.raw):
        h.engine.runner.free_request(key)
    h.raw.clear()
    h.engine = None
