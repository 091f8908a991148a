"""One registry from an architecture's name to its model.

The reference registers a creator per architecture by static initialisation
(``REGISTER_MODULE_OBJECT(QWen3Creator, ModelCreatorBase, "MODELCreator",
"qwen3")``, src/core/model/qwen3/QWen3Creator.cpp:11-12) and looks it up by
the file's architecture string (src/core/runtime/InferRuntime.cu:42-47),
logging and returning null on a miss; here a miss is an error that lists the
known names.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass

import torch

from ..config.base import ConfigError, ModelConfig
from ..weights.safetensors_io import load_model_dir
from .decoder import DecoderModel, TensorNames


@dataclass
class Architecture:
    name: str
    config_cls: type
    names: TensorNames
    model_cls: type = DecoderModel


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: type, names: TensorNames,
                          model_cls: type = DecoderModel) -> Architecture:
    arch = Architecture(name, config_cls, names, model_cls)
    _ARCHITECTURES[name] = arch
    return arch


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"architecture '{name}' is not registered; known: {sorted(_ARCHITECTURES)}") from None


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def config_from_dict(d: dict) -> ModelConfig:
    archs = d.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: required key 'architectures' (a list of names) is missing")
    return get_architecture(archs[0]).config_cls.from_dict(d)


def load_config(model_dir: str) -> ModelConfig:
    path = os.path.join(model_dir, "config.json")
    if not os.path.exists(path):
        raise ConfigError(f"{model_dir}: no config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except ValueError as e:
        raise ConfigError(f"{path}: not valid JSON: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return config_from_dict(d)


def build_model_skeleton(config: ModelConfig) -> DecoderModel:
    """The model's parts without weights (no device is touched)."""
    arch = get_architecture(config.architecture)
    return arch.model_cls(config, arch.names)


def load_model(model_dir: str, dtype: torch.dtype, device="cuda:0") -> DecoderModel:
    """Model of the folder's config.json with the folder's weights on ``device``
    in ``dtype`` (float32: everything widened to 32 bits; bfloat16: matrices in
    bfloat16, norm weights in float32)."""
    config = load_config(model_dir)
    model = build_model_skeleton(config)
    found = load_model_dir(model_dir)
    model.load_tensors(found, dtype, device, where=model_dir)
    return model
