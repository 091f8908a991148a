import json
import os
import struct

import pytest
import torch

from helpers import TINY_A, TINY_B, make_model_dir
from tffinfer_amd.models import build_model_skeleton, config_from_dict
from tffinfer_amd.weights import (WeightError, WeightFileError, check_weights, load_file, load_model_dir,
                                  normalize_stored, save_file, write_random_model)


def test_round_trip_bytes(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16),
         "c": torch.arange(6, dtype=torch.int64).reshape(2, 3), "d": torch.randn(2, 2).to(torch.float16)}
    p = str(tmp_path / "x.safetensors")
    save_file(t, p)
    back = load_file(p)
    assert set(back) == set(t)
    for k in t:
        assert back[k].dtype == t[k].dtype and torch.equal(back[k], t[k])


def test_matches_the_safetensors_library(tmp_path):
    from safetensors.torch import load_file as lib_load, save_file as lib_save
    t = {"w": torch.randn(4, 6).to(torch.bfloat16), "n": torch.randn(6)}
    save_file(t, str(tmp_path / "mine.safetensors"))
    theirs = lib_load(str(tmp_path / "mine.safetensors"))
    assert all(torch.equal(theirs[k], t[k]) for k in t)
    lib_save(t, str(tmp_path / "theirs.safetensors"))
    mine = load_file(str(tmp_path / "theirs.safetensors"))
    assert all(torch.equal(mine[k], t[k]) for k in t)


def test_stored_types_are_kept():
    assert normalize_stored(torch.zeros(2, dtype=torch.bfloat16)).dtype == torch.bfloat16
    assert normalize_stored(torch.zeros(2, dtype=torch.float32)).dtype == torch.float32
    assert normalize_stored(torch.zeros(2, dtype=torch.int64)).dtype == torch.int32
    assert normalize_stored(torch.zeros(2, dtype=torch.float16)).dtype == torch.float32


def test_random_model_folder(tmp_path):
    d = make_model_dir(str(tmp_path / "m"), TINY_B, 5)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    cfg = json.load(open(os.path.join(d, "config.json")))
    assert cfg["architectures"] == ["Qwen3ForCausalLM"] and cfg["intermediate_size"] == 200
    t = load_model_dir(d)
    model = build_model_skeleton(config_from_dict(cfg))
    check_weights(model.expected_tensors(), t)
    assert t["lm_head.weight"].shape == (320, 96)
    assert t["model.layers.2.self_attn.q_proj.weight"].shape == (256, 96)
    assert t["model.layers.0.self_attn.q_norm.weight"].dtype == torch.float32
    assert t["model.layers.0.mlp.down_proj.weight"].dtype == torch.bfloat16
    w = t["model.layers.1.mlp.up_proj.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    n = torch.cat([t[k].float() for k in t if k.endswith("layernorm.weight")])
    assert abs(float(n.mean()) - 1.0) < 0.05 and 0.05 < float(n.std()) < 0.15
    # same seed, same bytes; another seed, other bytes; tied model has no head tensor
    d2 = make_model_dir(str(tmp_path / "m2"), TINY_B, 5)
    assert all(torch.equal(load_model_dir(d2)[k], t[k]) for k in t)
    d3 = make_model_dir(str(tmp_path / "m3"), TINY_B, 6)
    assert not torch.equal(load_model_dir(d3)["lm_head.weight"], t["lm_head.weight"])
    ta = load_model_dir(make_model_dir(str(tmp_path / "a"), TINY_A, 1))
    assert "lm_head.weight" not in ta


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = make_model_dir(str(tmp_path / "m"), TINY_A, 5)
    t = dict(load_model_dir(d))
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64, dtype=torch.bfloat16)
    t["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(16, dtype=torch.int32)
    model = build_model_skeleton(config_from_dict(TINY_A))
    with pytest.raises(WeightError) as ei:
        model.load_tensors(t, torch.float32, "cpu")
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert e.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (64, 64))]
    assert e.wrong_dtype == [("model.layers.0.self_attn.q_norm.weight", torch.int32)]
    msg = str(e)
    for piece in ("missing (2)", "unexpected (1)", "expected [32, 64], found [64, 64]", "rotary_emb"):
        assert piece in msg


def test_tied_model_ignores_a_stored_head(tmp_path):
    d = make_model_dir(str(tmp_path / "m"), TINY_A, 5)
    t = dict(load_model_dir(d))
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    model = build_model_skeleton(config_from_dict(TINY_A))
    check_weights(model.expected_tensors(), t, {"lm_head.weight"})
    # the model says so when it passes a stored copy over
    import io
    from tffinfer_amd import log
    buf = io.StringIO()
    level, app, stream = log.get_level(), log._State.app, log._State.stream
    log.init("unit", "info", buf)
    try:
        model.load_tensors(t, torch.float32, "cpu", where=d)
    finally:
        log.init(app, level, stream)
    assert "lm_head.weight" in buf.getvalue() and buf.getvalue().startswith("W")


def test_broken_files(tmp_path):
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(WeightFileError, match="too short"):
        load_file(str(p))
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(WeightFileError, match="header length"):
        load_file(str(p))
    p.write_bytes(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(WeightFileError, match="JSON"):
        load_file(str(p))
    good = str(tmp_path / "g.safetensors")
    save_file({"w": torch.randn(8, 8)}, good)
    raw = open(good, "rb").read()
    (tmp_path / "t.safetensors").write_bytes(raw[:-10])
    with pytest.raises(WeightFileError, match="truncated"):
        load_file(str(tmp_path / "t.safetensors"))
    hdr = json.dumps({"w": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}}).encode()
    (tmp_path / "u.safetensors").write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0\0")
    with pytest.raises(WeightFileError, match="unsupported dtype"):
        load_file(str(tmp_path / "u.safetensors"))
    with pytest.raises(WeightFileError, match="neither"):
        load_model_dir(str(tmp_path / "empty_dir_that_is_missing"))
    # a tensor named twice in the header (a JSON parser keeps the last without a word)
    hdr = (b'{"w": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}, '
           b'"w": {"dtype": "F32", "shape": [1], "data_offsets": [4, 8]}}')
    (tmp_path / "d.safetensors").write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(WeightFileError, match="more than once"):
        load_file(str(tmp_path / "d.safetensors"))


def test_sharded_folder(tmp_path):
    d = tmp_path / "s"
    d.mkdir()
    save_file({"a": torch.ones(2)}, str(d / "model-00001-of-00002.safetensors"))
    save_file({"b": torch.zeros(3)}, str(d / "model-00002-of-00002.safetensors"))
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {
        "a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors"}}))
    t = load_model_dir(str(d))
    assert set(t) == {"a", "b"}
