from .base import ConfigError
from .qwen3 import Qwen3Config
from .registry import (Architecture, detect_architecture, known_architectures, load_model_config,
                       register_architecture)

__all__ = ["ConfigError", "Qwen3Config", "Architecture", "detect_architecture",
           "known_architectures", "load_model_config", "register_architecture"]
