"""A small inference engine for the Qwen3 dense decoder on one MI355X."""
from . import parts  # registers the built-in parts
from . import models  # registers the architecture
from .config import ConfigError, Qwen3Config
from .models import load_config, load_model, register_architecture

__version__ = "0.1.0"
