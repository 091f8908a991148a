import json

import pytest

from helpers import TINY_A, TINY_B
from tffinfer_amd.config import ConfigError, Qwen3Config
from tffinfer_amd.models import (config_from_dict, get_architecture, load_config,
                                 registered_architectures)


def test_reads_every_key():
    c = Qwen3Config.from_dict(TINY_B)
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads) == (96, 3, 8, 2)
    assert (c.head_dim, c.intermediate_size, c.vocab_size, c.max_position_embeddings) == (32, 200, 320, 256)
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 1e6 and c.tie_word_embeddings is False
    assert c.layer_windows() == [0, 24, 24]


def test_defaults():
    d = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "head_dim", "rms_norm_eps",
                                                      "rope_theta", "tie_word_embeddings")}
    c = Qwen3Config.from_dict(d)
    assert c.num_key_value_heads == c.num_attention_heads == 4
    assert c.head_dim == 16 and c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0
    assert c.tie_word_embeddings is False


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "intermediate_size", "vocab_size", "max_position_embeddings"])
def test_missing_key_is_an_error(key):
    d = dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(d)


@pytest.mark.parametrize("patch,match", [
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"attention_bias": True}, "attention_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"hidden_size": "64"}, "integer"),
    ({"vocab_size": 0}, "positive"),
    ({"layer_types": ["full_attention"]}, "layer_types"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, "window"),
])
def test_inconsistent_or_unsupported(patch, match):
    with pytest.raises(ConfigError, match=match):
        Qwen3Config.from_dict({**TINY_A, **patch})


def test_registry():
    assert "Qwen3ForCausalLM" in registered_architectures()
    assert get_architecture("Qwen3ForCausalLM").config_cls is Qwen3Config
    with pytest.raises(ConfigError, match="Qwen3ForCausalLM"):   # the error lists the known names
        get_architecture("LlamaForCausalLM")
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({"hidden_size": 8})
    assert isinstance(config_from_dict(TINY_A), Qwen3Config)


def test_load_config_from_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    c = load_config(str(tmp_path))
    assert c.num_hidden_layers == 3
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path / "nowhere"))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))


def test_round_trip_and_layer_data():
    c = Qwen3Config.from_dict(TINY_B)
    again = Qwen3Config.from_dict(c.to_dict())
    assert again.layer_windows() == c.layer_windows() and again.head_dim == c.head_dim
    specs = c.layer_specs()
    assert len(specs) == 3
    assert [s.mixer.args["window"] for s in specs] == [0, 24, 24]
    assert specs[0].mixer.kind == "gqa_attention" and specs[0].feed_forward.kind == "swiglu"
    assert specs[0].norm.args["eps"] == 1e-5
    sched = c.layer_schedule()
    assert [(s.layer, s.cache, s.writes_cache) for s in sched] == [(0, 0, True), (1, 1, True), (2, 2, True)]


def test_a_model_of_built_in_parts_is_one_graph_piece():
    """Every built-in part can be captured, so a decode step is one piece: embedding, every
    entry of the run order, final norm and head."""
    from helpers import TINY_B
    from tffinfer_amd.models import build_model_skeleton, config_from_dict
    model = build_model_skeleton(config_from_dict(dict(TINY_B)))
    assert model.graph_safe()
    assert model.graph_pieces() == [(True, ["embed", 0, 1, 2, "finish"])]
