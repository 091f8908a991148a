"""Shared by the tests: the tiny configurations, model folders, the oracle."""
from __future__ import annotations

import functools
import json
import os

import torch

# Two tiny configurations that differ in every size and option.
TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=64, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128,
    vocab_size=256, max_position_embeddings=128, rms_norm_eps=1e-6, rope_theta=10000.0,
    tie_word_embeddings=True, use_sliding_window=False,
)
TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=96, num_hidden_layers=3,
    num_attention_heads=8, num_key_value_heads=2, head_dim=32, intermediate_size=200,
    vocab_size=320, max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=1000000.0,
    tie_word_embeddings=False, use_sliding_window=True, sliding_window=24, max_window_layers=1,
)
# A third one with the head size of the large models, an odd group size and sizes that are
# multiples of 8 only.
TINY_C = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=168, num_hidden_layers=2,
    num_attention_heads=5, num_key_value_heads=1, head_dim=128, intermediate_size=136,
    vocab_size=1000, max_position_embeddings=512, rms_norm_eps=3e-6, rope_theta=500000.0,
    tie_word_embeddings=False,
)
# The same head size with a sliding window on every other layer (the decode kernel that writes
# keys itself, on pages that a window has passed and given back), four heads to a kv head.
TINY_D = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=104, num_hidden_layers=4,
    num_attention_heads=4, num_key_value_heads=1, head_dim=64, intermediate_size=72,
    vocab_size=777, max_position_embeddings=320, rms_norm_eps=2e-6, rope_theta=20000.0,
    tie_word_embeddings=True, use_sliding_window=True, sliding_window=40, max_window_layers=2,
)
# B with full attention in all three layers (a q projection wider than the hidden size over a
# cache that keeps every key, pages of 8 tokens).
TINY_B0 = dict(TINY_B, use_sliding_window=False)
# Eight kv heads: with twenty decoding requests and more a decode step gives every (request, kv
# head) pair a block of waves of its own, and products of 17 to 64 rows run on tiles that split K.
TINY_E = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=128, num_hidden_layers=2,
    num_attention_heads=16, num_key_value_heads=8, head_dim=64, intermediate_size=176,
    vocab_size=500, max_position_embeddings=512, rms_norm_eps=5e-6, rope_theta=300000.0,
    tie_word_embeddings=False,
)
# The same with rows wide enough that every product of 17 to 64 rows splits K (the fused q, k, v
# projection and the gated product included), and the head size of the large models.
TINY_W = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=1024, num_hidden_layers=2,
    num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=2112,
    vocab_size=1200, max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=1000000.0,
    tie_word_embeddings=True,
)
TINY_CONFIGS = {"A": (TINY_A, 11), "B": (TINY_B, 23), "C": (TINY_C, 31), "D": (TINY_D, 47), "B0": (TINY_B0, 23),
                "E": (TINY_E, 53), "W": (TINY_W, 59)}
PAGE_SIZE = {"A": 16, "B": 8, "C": 32, "D": 16, "B0": 8, "E": 16, "W": 16}


def make_model_dir(path: str, cfg: dict, seed: int, dtype: str = "bfloat16") -> str:
    from tffinfer_amd.weights import write_random_model
    write_random_model(path, dict(cfg), seed, dtype=dtype)
    return path


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


@functools.lru_cache(maxsize=64)
def _oracle_cached(model_dir: str, tokens: tuple) -> torch.Tensor:
    from plain_qwen3 import fast_forward, load_plain_model
    cfg, raw = load_plain_model(model_dir, torch.float64)
    return fast_forward(cfg, raw, list(tokens))


def oracle_logits(model_dir: str, tokens) -> torch.Tensor:
    """float64 logits [T, V] of the plain implementation for a whole sequence."""
    return _oracle_cached(model_dir, tuple(int(t) for t in tokens))


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest absolute difference over the largest reference magnitude."""
    got = got.double().cpu()
    ref = ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# Tolerances on rel_err, per configuration: about twice the worst error seen over all the ways
# of cutting and batching (float32: 4.1e-7 / 1.0e-6 / 1.2e-6 / 8.8e-7 for A / B / C / D, 1.3e-6 / 3.5e-6
# for E / W and 5.7e-6 at the middle size; bfloat16: 4.6e-3 / 9.1e-3 / 8.8e-3 / 8.3e-3, 7.3e-3 / 1.3e-2
# and 1.3e-2; a run prints what it saw at its end).
# float32: the engine differs from a float64 run by rounding only.  bfloat16: weights are the
# same bfloat16 values in both runs; the engine rounds activations to bfloat16 between kernels
# (relative step 2^-8).  One wrong page among a request's five moves the logits of these models
# by 7e-2 and more.
_TOL = {
    "float32": {"A": 1e-6, "B": 2.5e-6, "C": 3e-6, "D": 2e-6, "B0": 2.5e-6, "E": 3e-6, "W": 7e-6, "mid": 1.2e-5,
                "large": 1.2e-5},
    "bfloat16": {"A": 1e-2, "B": 2e-2, "C": 1.8e-2, "D": 1.6e-2, "B0": 2e-2, "E": 1.5e-2, "W": 2.6e-2, "mid": 2.6e-2,
                 "large": 2e-2},
}


#: the worst rel_err seen in this run per (dtype, configuration) by the comparisons with the oracle;
#: printed at the end of a run (conftest), so that the tolerances can be held against it
WORST: dict = {}


def note_error(dtype: str, name: str, err: float) -> None:
    key = (dtype, os.path.basename(os.path.normpath(name)))
    if err > WORST.get(key, 0.0):
        WORST[key] = err


def tol(dtype: str, name: str) -> float:
    """Tolerance for configuration ``name`` (or a model folder named after it)."""
    return _TOL[dtype][os.path.basename(os.path.normpath(name))]


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)
