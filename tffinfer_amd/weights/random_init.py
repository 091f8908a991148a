"""Seeded random weights, and writing a model folder from a configuration."""
from __future__ import annotations

import hashlib
import json
import os

import torch

from ..parts.base import WeightSpec
from .safetensors_io import save_file

MATRIX_STD = 0.02
NORM_STD = 0.1


def tensor_seed(seed: int, name: str) -> int:
    """A seed per tensor, so values do not depend on the order of creation."""
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(spec: WeightSpec, seed: int, name: str, device="cpu") -> torch.Tensor:
    """float32 values: matrices and embeddings N(0, 0.02), norm weights
    1 + N(0, 0.1)."""
    g = torch.Generator(device=device)
    g.manual_seed(tensor_seed(seed, name))
    x = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
    if spec.init == "norm":
        return 1.0 + NORM_STD * x
    return MATRIX_STD * x


def write_random_model(model_dir: str, config, seed: int, dtype: str = "bfloat16") -> str:
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (a typed
    configuration or a config.json dict) with weights drawn from ``seed``.
    Matrices are stored in ``dtype``; norm weights always in float32."""
    from ..models.registry import build_model_skeleton, config_from_dict
    if isinstance(config, dict):
        config = config_from_dict(config)
    store = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    expected = build_model_skeleton(config).expected_tensors()
    tensors = {}
    for name, spec in expected.items():
        t = random_tensor(spec, seed, name)
        tensors[name] = t if spec.init == "norm" else t.to(store)
    os.makedirs(model_dir, exist_ok=True)
    d = config.to_dict()
    d["torch_dtype"] = dtype
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(d, f, indent=2)
    save_file(tensors, os.path.join(model_dir, "model.safetensors"),
              metadata={"format": "pt", "seed": seed})
    return model_dir
