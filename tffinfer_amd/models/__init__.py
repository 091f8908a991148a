from . import qwen3  # noqa: F401  (registers the architecture)
from .decoder import DecoderModel, TensorNames
from .registry import (Architecture, build_model_skeleton, config_from_dict, get_architecture,
                       load_config, load_model, register_architecture, registered_architectures)
