"""The byte and flop counts of the measurements come from the model's own parts; here against
the closed formulas of the architecture, on model skeletons without weights."""
import pytest

from helpers import TINY_A, TINY_B, TINY_D
from tffinfer_amd import measure as M
from tffinfer_amd.models import build_model_skeleton, config_from_dict


def _sizes(c):
    return (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"],
            c["intermediate_size"], c["vocab_size"], c["num_hidden_layers"])


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_D], ids=["A", "B", "D"])
def test_counts_follow_the_parts(cfg):
    from plain_qwen3 import layer_windows
    H, nq, nkv, d, I, V, L = _sizes(cfg)
    model = build_model_skeleton(config_from_dict(cfg))
    per_layer = (nq + 2 * nkv) * d * H + nq * d * H + 3 * I * H
    assert M.matrix_elements_per_step(model) == per_layer * L
    windows = layer_windows(cfg)          # 0: the layer keeps every key
    batch, ctx, T = 3, 100, 90
    kv = sum(2 * nkv * d * 2 * batch * (min(ctx, w) if w else ctx) for w in windows)
    assert M.decode_bytes(model, batch, ctx) == (per_layer * L + H * V) * 2 + kv
    pairs = sum(sum(min(t + 1, w) if w else t + 1 for t in range(T)) for w in windows)
    assert M.prefill_flops(model, T) == pytest.approx(2.0 * T * per_layer * L + 4 * nq * d * pairs + 2.0 * H * V)
