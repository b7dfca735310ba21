from .base import (ConfigError, ModelConfig, load_config, lookup_architecture,
                   register_architecture, registered_architectures)
from .engine import EngineConfig
from .qwen3 import Qwen3Config

__all__ = ["ConfigError", "ModelConfig", "load_config", "lookup_architecture",
           "register_architecture", "registered_architectures", "EngineConfig", "Qwen3Config"]
