"""The engine's C interface (tffinfer_amd/csrc/tffinfer_engine.h), called the way a C program
calls it: through the shared library, with C structs and buffers.  In this process the library
uses the running interpreter; the example program (examples/engine_demo.c) starts its own.
The reference's manner: include/ExportInc.h:6-16, src/core/runtime/InferRuntime.h:32-45,
example/load_model/load_model.cu:8-25."""
import ctypes
import json
import os
import re
import subprocess

import numpy as np
import pytest
import torch

from helpers import TINY_A, TINY_B, make_model_dir, oracle_logits, random_tokens, rel_err, tol
from plain_qwen3 import plain_greedy

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "tffinfer_amd", "csrc", "tffinfer_engine.h")


class StepEvent(ctypes.Structure):
    _fields_ = [("request_id", ctypes.c_int64), ("token", ctypes.c_int32), ("finished", ctypes.c_int32)]


class RawEntry(ctypes.Structure):
    _fields_ = [("request_id", ctypes.c_int64), ("tokens", ctypes.POINTER(ctypes.c_int32)), ("n_tokens", ctypes.c_int32),
                ("want", ctypes.POINTER(ctypes.c_int32)), ("n_want", ctypes.c_int32)]


@pytest.fixture(scope="module")
def capi():
    from tffinfer_amd.kernels.build import build_engine_capi, find_engine_library
    path = find_engine_library() or build_engine_capi(verbose=False)
    L = ctypes.CDLL(path)
    P, I, I64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
    L.engine_create.restype = P
    L.engine_create.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    L.engine_create_random.restype = P
    L.engine_create_random.argtypes = [ctypes.c_char_p, ctypes.c_uint64, ctypes.c_char_p]
    L.engine_destroy.argtypes = [P]
    L.engine_destroy.restype = None
    L.engine_vocab_size.argtypes = [P]
    L.engine_add_request.restype = I64
    L.engine_add_request.argtypes = [P, ctypes.POINTER(ctypes.c_int32), ctypes.c_int32, ctypes.c_char_p]
    L.engine_step.argtypes = [P, ctypes.POINTER(StepEvent), I]
    L.engine_has_work.argtypes = [P]
    L.engine_abort.argtypes = [P, I64]
    L.engine_step_raw.argtypes = [P, ctypes.POINTER(RawEntry), I, ctypes.POINTER(ctypes.c_float), I64]
    L.engine_end_raw.argtypes = [P, I64]
    L.engine_last_error.restype = ctypes.c_char_p
    return L


def ids_array(ids):
    return (ctypes.c_int32 * len(ids))(*ids)


def run_all(L, e, capacity=16):
    """Steps until nothing is left; tokens per request id, and the ids that finished."""
    out, done = {}, []
    ev = (StepEvent * capacity)()
    while L.engine_has_work(e) == 1:
        n = L.engine_step(e, ev, capacity)
        assert n >= 0, L.engine_last_error()
        for x in ev[:n]:
            if x.token >= 0:
                out.setdefault(x.request_id, []).append(x.token)
            if x.finished:
                done.append(x.request_id)
    return out, done


# ---- without a GPU -------------------------------------------------------------
def test_header_and_library_agree(capi):
    """Every function the header declares is exported, and nothing else of the library's is."""
    text = open(HEADER).read()
    declared = set(re.findall(r"TFF_ENGINE_API\s+[\w\s\*]+?\b(engine_\w+)\s*\(", text))
    assert declared == {"engine_create", "engine_create_random", "engine_destroy", "engine_vocab_size",
                        "engine_add_request", "engine_step", "engine_has_work", "engine_abort", "engine_step_raw",
                        "engine_end_raw", "engine_last_error"}
    for name in declared:
        assert hasattr(capi, name), name
    from tffinfer_amd.kernels.build import find_engine_library
    syms = subprocess.run(["nm", "-D", "--defined-only", find_engine_library()], capture_output=True, text=True).stdout
    exported = {ln.split()[-1] for ln in syms.splitlines() if " T " in ln}
    assert exported == declared, exported ^ declared


def test_errors_come_back_as_messages(capi, tmp_path):
    assert capi.engine_last_error() == b""
    assert capi.engine_create(str(tmp_path / "nowhere").encode(), None) is None
    assert b"nowhere" in capi.engine_last_error()
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(TINY_A))
    assert capi.engine_create_random(str(cfg).encode(), 1, b'{"pages": 3}') is None
    assert b"unknown keys ['pages']" in capi.engine_last_error()
    assert capi.engine_create_random(str(cfg).encode(), 1, b'[1, 2]') is None
    assert b"JSON object" in capi.engine_last_error()
    assert capi.engine_add_request(None, ids_array([1]), 1, None) == -1
    assert b"engine_add_request" in capi.engine_last_error()
    assert capi.engine_has_work(None) == -1 and capi.engine_step(None, (StepEvent * 1)(), 1) == -1
    capi.engine_destroy(None)       # harmless


# ---- on the GPU ----------------------------------------------------------------
@pytest.mark.gpu
def test_generation_through_the_c_interface(capi, tmp_path):
    """Requests and steps through C structs give the tokens that the plain implementation
    chooses from its own logits; an event buffer of one event loses nothing; an aborted
    request ends with an event and gives its pages back."""
    folder = make_model_dir(str(tmp_path / "A"), TINY_A, 11, dtype="float32")
    e = capi.engine_create(folder.encode(), b'{"dtype": "float32", "max_model_len": 128, "kv_tokens": 512, "page_size": 16}')
    assert e, capi.engine_last_error()
    assert capi.engine_vocab_size(e) == TINY_A["vocab_size"]
    prompts = [random_tokens(n, TINY_A["vocab_size"], 300 + n) for n in (5, 33, 70)]
    params = b'{"max_new_tokens": 9, "ignore_eos": true}'
    rids = [capi.engine_add_request(e, ids_array(p), len(p), params) for p in prompts]
    assert rids == [0, 1, 2], capi.engine_last_error()
    out, done = run_all(capi, e, capacity=1)
    assert sorted(done) == rids
    for rid, p in zip(rids, prompts):
        seq = p + out[rid]
        ref = oracle_logits(folder, seq)
        assert len(out[rid]) == 9
        assert out[rid] == [plain_greedy(ref[len(p) - 1 + j]) for j in range(9)]
    # a token outside the vocabulary is refused with a message, and the engine goes on
    assert capi.engine_add_request(e, ids_array([1, 9999]), 2, params) == -1
    assert b"vocabulary" in capi.engine_last_error()
    # abort: one of two requests, before its first step
    a = capi.engine_add_request(e, ids_array(prompts[0]), len(prompts[0]), params)
    b = capi.engine_add_request(e, ids_array(prompts[1]), len(prompts[1]), b'{"max_new_tokens": 3, "ignore_eos": true, "sampling": {"type": "top_k", "top_k": 1, "temperature": 0.7, "seed": 5}}')
    assert capi.engine_abort(e, a) == 1 and capi.engine_abort(e, 12345) == 0
    out2, done2 = run_all(capi, e)
    assert a not in out2 and out2[b] == out[rids[1]][:3]        # top_k of one is greedy
    capi.engine_destroy(e)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_raw_steps_through_the_c_interface(capi, tmp_path, dtype):
    """engine_step_raw: portions of one request beside single tokens of another, logits at the
    wanted places against the plain implementation; pages come back with engine_end_raw."""
    folder = make_model_dir(str(tmp_path / "B"), TINY_B, 23)
    V = TINY_B["vocab_size"]
    opts = json.dumps({"dtype": dtype, "max_model_len": 256, "num_pages": 16, "page_size": 8}).encode()
    e = capi.engine_create(folder.encode(), opts)
    assert e, capi.engine_last_error()
    a, b = random_tokens(61, V, 1), random_tokens(40, V, 2)
    ra, rb = oracle_logits(folder, a), oracle_logits(folder, b)
    buf = (ctypes.c_float * (8 * V))()

    def raw(entries):
        arr = (RawEntry * len(entries))()
        keep = []
        for i, (rid, toks, want) in enumerate(entries):
            t, w = ids_array(toks), ids_array(want)
            keep += [t, w]
            arr[i] = RawEntry(rid, t, len(toks), w, len(want))
        n = capi.engine_step_raw(e, arr, len(entries), buf, len(buf))
        assert n >= 0, capi.engine_last_error()
        return torch.from_numpy(np.ctypeslib.as_array(buf)[: n * V].reshape(n, V).copy())

    worst = 0.0
    got = raw([(7, a[:30], [0, 29]), (9, b[:2], [])])
    worst = max(worst, rel_err(got[0], ra[0]), rel_err(got[1], ra[29]))
    got = raw([(9, b[2:39], [36]), (7, a[30:31], [0])])
    worst = max(worst, rel_err(got[0], rb[38]), rel_err(got[1], ra[30]))
    got = raw([(7, a[31:], [0, 29]), (9, b[39:], [0])])
    worst = max(worst, rel_err(got[0], ra[31]), rel_err(got[1], ra[60]), rel_err(got[2], rb[39]))
    assert worst <= tol(dtype, "B"), worst
    # too little room is refused before anything runs
    arr = (RawEntry * 1)(RawEntry(7, ids_array([1]), 1, ids_array([0]), 1))
    assert capi.engine_step_raw(e, arr, 1, buf, V - 1) == -1 and b"do not fit" in capi.engine_last_error()
    # 61 + 40 tokens hold 8 + 5 pages of the 16: a third request of 60 tokens fits only once they are given back
    c = random_tokens(60, V, 3)
    arr = (RawEntry * 1)(RawEntry(11, ids_array(c), len(c), ids_array([59]), 1))
    assert capi.engine_step_raw(e, arr, 1, buf, len(buf)) == -1
    assert capi.engine_end_raw(e, 11) == 1      # (opened by the failed step)
    assert capi.engine_end_raw(e, 7) == 1 and capi.engine_end_raw(e, 7) == 0 and capi.engine_end_raw(e, 9) == 1
    got = raw([(11, c, [59])])
    assert rel_err(got[0], oracle_logits(folder, c)[59]) <= tol(dtype, "B")
    capi.engine_destroy(e)


@pytest.mark.gpu
def test_example_program_starts_its_own_interpreter(tmp_path):
    """examples/engine_demo.c, a C program with no Python of its own: random weights from a
    config file and a seed are those of the folder that the weights module writes."""
    from tffinfer_amd.kernels.build import find_engine_library
    demo = os.path.join(os.path.dirname(find_engine_library()), "engine_demo")
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(TINY_A))
    folder = make_model_dir(str(tmp_path / "A"), TINY_A, 77, dtype="float32")
    prompts = [[3, 14, 15, 92, 65], [200, 1]]
    env = dict(os.environ, TFF_ENGINE_OPTIONS='{"dtype": "float32", "max_model_len": 128, "kv_tokens": 256}')
    for source in (["--random", f"{cfg}:77"], [folder]):
        p = subprocess.run([demo, *source, "5", *[",".join(map(str, q)) for q in prompts]], capture_output=True,
                           text=True, timeout=300, env=env)
        assert p.returncode == 0, p.stderr[-3000:]
        lines = p.stdout.strip().splitlines()
        assert len(lines) == 2
        for i, q in enumerate(prompts):
            toks = [int(t) for t in lines[i].split(":")[1].split()]
            ref = oracle_logits(folder, q + toks)
            assert toks == [plain_greedy(ref[len(q) - 1 + j]) for j in range(5)]
    p = subprocess.run([demo, str(tmp_path / "nowhere"), "5", "1,2"], capture_output=True, text=True, timeout=300, env=env)
    assert p.returncode == 1 and "nowhere" in p.stderr
