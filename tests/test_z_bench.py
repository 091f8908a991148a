"""The benchmark program's contract: one JSON line of fixed keys at one GPU, a refusal for more."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_one_line():
    p = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "--gpus 2" in p.stdout


@pytest.mark.gpu
def test_one_json_line_with_the_contract_keys():
    """One layer of the benchmark shape, a short context beyond which the length limit need not
    grow, and a prompt longer than that limit (the limit grows with it)."""
    cmd = [sys.executable, BENCH, "--layers", "1", "--steps", "4", "--warmup", "2", "--batch", "2",
           "--context", "256", "--prefill-tokens", "8200"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = p.stdout.strip().splitlines()
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 4 and rec["warmup"] == 2 and rec["dtype"] == "bf16"
    assert rec["value"] == pytest.approx(2 * 1000.0 / rec["ms_per_step"], rel=1e-3)
    # the steps by device events: a median that the wall-clock mean cannot be far below
    assert 0 < rec["ms_per_step_median"] < 3 * rec["ms_per_step"]
    ceil = rec["ceilings"]
    assert 2000 < ceil["stream_read_GBps"] < 8000 and 500 < ceil["mfma_bf16_TFLOPs"] < 2500
    assert rec["roofline"]["frac_of_measured"] == pytest.approx(rec["roofline"]["achieved"] / ceil["stream_read_GBps"], abs=1e-3)
    assert rec["prefill"]["frac_of_measured"] == pytest.approx(rec["prefill"]["frac"] * 2500.0 / ceil["mfma_bf16_TFLOPs"], rel=2e-2)
    assert rec["prefill"]["ms_device"] <= rec["prefill"]["ms"] * 1.05
    cfg = rec["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 36 and cfg["layers_run"] == 1 and cfg["global_batch"] == 2 and cfg["seq_len"] == 256
    assert cfg["max_context"] == 16384   # grown from the shape's 8,192 to hold the 8,200-token prompt
    assert rec["prefill"]["tokens"] == 8200 and rec["prefill"]["ms"] > 0 and 0 < rec["prefill"]["frac"] < 1
    assert rec["roofline"]["bound"] == "hbm" and rec["roofline"]["peak"] == 8000.0
    assert rec["roofline"]["frac"] == pytest.approx(rec["roofline"]["achieved"] / 8000.0, abs=1e-3)
    assert set(rec["points"]) == {"decode_b1", "decode_b64", "decode_b2_top_k50_top_p0.95"}
    assert all(v > 0 for v in rec["points"].values())
    for key, b in (("decode_b1", 1), ("decode_b64", 64)):      # a point's own time and share of the HBM peak
        d = rec["points_detail"][key]
        assert rec["points"][key] == pytest.approx(b * 1000.0 / d["ms_per_step"], rel=1e-3)
        assert 0 < d["ms_per_step_median"] < 3 * d["ms_per_step"] and 0 < d["frac"] < 1
    assert rec["points"]["decode_b2_top_k50_top_p0.95"] < 1.05 * rec["value"]      # drawing costs something, not nothing
