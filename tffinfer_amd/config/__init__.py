from .base import ConfigError, LayerCall, LayerSpec, ModelConfig, PartSpec
from .qwen3 import Qwen3Config
