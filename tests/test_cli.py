"""The command line's options, each through a subprocess as a user calls it
(the reference's manner: test/main.cu:17-66, example/load_model/load_model.cu:8-25)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from helpers import TINY_A, TINY_B, oracle_logits, random_tokens, rel_err, tol
from plain_qwen3 import plain_greedy

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROG = os.path.join(ROOT, "bin", "tffinfer")


def run(*args, timeout=300):
    return subprocess.run([sys.executable, PROG, *map(str, args)], capture_output=True, text=True, timeout=timeout)


def config_file(tmp_path, cfg, name="config.json"):
    path = tmp_path / name
    path.write_text(json.dumps(cfg))
    return str(path)


# ---- refusals, no GPU needed -------------------------------------------------
def test_neither_model_nor_config():
    p = run("--prompt-ids", "1,2")
    assert p.returncode == 2 and "model folder, or --config" in p.stderr


def test_config_without_random_weights(tmp_path):
    p = run("--config", config_file(tmp_path, TINY_A), "--prompt-ids", "1,2")
    assert p.returncode == 2 and "--random-weights" in p.stderr


def test_no_other_device(tmp_path):
    p = run("--config", config_file(tmp_path, TINY_A), "--random-weights", "--device", "cpu-ref")
    assert p.returncode == 2 and "no CPU path" in p.stderr


def test_one_way_to_size_the_cache(tmp_path):
    p = run("--config", config_file(tmp_path, TINY_A), "--random-weights", "--num-pages", "4", "--kv-bytes", "4096")
    assert p.returncode == 2 and "one of" in p.stderr


def test_log_level_off_is_silent(tmp_path):
    p = run("--prompt-ids", "1,2", "--log-level", "off")
    assert p.returncode == 2 and p.stderr == ""


# ---- on the GPU --------------------------------------------------------------
@pytest.mark.gpu
def test_random_weights_from_a_config_file_and_dumped_logits(tmp_path):
    """--config FILE --random-weights --seed N: the weights are those of the folder that
    --save-model writes; the dumped rows are the logits that chose each token."""
    cfg = config_file(tmp_path, TINY_B)
    folder = str(tmp_path / "B")
    prompts = [random_tokens(n, TINY_B["vocab_size"], 900 + n) for n in (7, 30)]
    dump = str(tmp_path / "logits.f32")
    args = ["--config", cfg, "--random-weights", "--seed", "23", "--save-model", folder, "--fp32", "--n-ctx", "256",
            "--n-predict", "6", "--ignore-eos", "--json", "--dump-logits", dump]
    for pr in prompts:
        args += ["--prompt-ids", ",".join(map(str, pr))]
    p = run(*args)
    assert p.returncode == 0, p.stderr[-3000:]
    recs = [json.loads(ln) for ln in p.stdout.strip().splitlines()]
    assert [r["prompt"] for r in recs] == prompts
    meta = json.load(open(dump + ".json"))
    V = TINY_B["vocab_size"]
    assert meta["shape"] == [12, V] and [r["rows"] for r in meta["requests"]] == [6, 6]
    rows = np.fromfile(dump, dtype="<f4").reshape(12, V)
    import torch
    for i, r in enumerate(recs):
        seq = r["prompt"] + r["output"]
        ref = oracle_logits(folder, seq)
        first = meta["requests"][i]["first_row"]
        assert meta["requests"][i]["first_position"] == len(r["prompt"]) - 1
        for j, tok in enumerate(r["output"]):
            row = torch.from_numpy(rows[first + j].copy())
            assert rel_err(row, ref[len(r["prompt"]) - 1 + j]) <= tol("float32", "B")
            assert tok == plain_greedy(row)


@pytest.mark.gpu
@pytest.mark.parametrize("how", ["num-pages", "kv-bytes"])
def test_cache_geometry_options(tmp_path, how):
    """A pool of 9 pages of 8 tokens, given as pages and as bytes: the requests do not fit
    together, are preempted, and give the tokens they give with room for all."""
    cfg = config_file(tmp_path, TINY_A)
    common = ["--config", cfg, "--random-weights", "--seed", "11", "--fp32", "--n-ctx", "128", "--n-predict", "20",
              "--ignore-eos", "--json", "--random-prompts", "3:30", "--page-size", "8", "--max-batches", "3"]
    roomy = run(*common, "--kv-tokens", "512")
    assert roomy.returncode == 0, roomy.stderr[-3000:]
    # a page of 8 tokens: 2 layers x (K and V) x 2 kv heads x 16 x 8 tokens x 4 bytes
    per_page = 2 * 2 * 2 * 16 * 8 * 4
    size = ["--num-pages", "9"] if how == "num-pages" else ["--kv-bytes", str(9 * per_page + 100)]
    tight = run(*common, *size)
    assert tight.returncode == 0, tight.stderr[-3000:]
    assert tight.stdout == roomy.stdout
    assert "0 preemptions" in roomy.stderr and "preemptions" in tight.stderr and "0 preemptions" not in tight.stderr


@pytest.mark.gpu
def test_kv_bytes_below_one_page_is_an_error(tmp_path):
    p = run("--config", config_file(tmp_path, TINY_A), "--random-weights", "--kv-bytes", "100", "--prompt-ids", "1")
    assert p.returncode != 0 and "holds no page" in p.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("phase", ["decode", "prefill"])
def test_bench_mode(tmp_path, phase):
    cfg = dict(TINY_A, max_position_embeddings=512)
    p = run("--config", config_file(tmp_path, cfg), "--random-weights", "--bench", phase, "--batch", "3",
            "--context", "96", "--gen", "5")
    assert p.returncode == 0, p.stderr[-3000:]
    rec = json.loads(p.stdout.strip().splitlines()[-1])
    assert rec["bench"] == phase and rec["context"] == 96 and rec["tokens_per_s"] > 0
    if phase == "decode":
        assert rec["steps"] == 5 and rec["ms_per_step"] > 0 and rec["ms_per_step_median"] > 0 and 0 < rec["hbm_frac"] < 1
    else:
        assert rec["ms"] > 0 and rec["ms_device"] > 0 and 0 <= rec["mfma_frac"] < 1
