"""A small inference engine for the Qwen3 dense decoder on one MI355X."""
from . import parts  # registers the built-in parts
from . import models  # registers the architecture
from .config import ConfigError, Qwen3Config
from .engine import EngineOptions, LLMEngine, ModelRunner, StepEntry
from .models import load_config, load_model, register_architecture
from .runtime import LLMInferRuntime, ModelConfig
from .sampling import SamplingConfig

__version__ = "0.1.0"
