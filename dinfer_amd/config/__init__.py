from .base import ConfigError, ModelConfig, key
from .options import EngineOptions
from .registry import (Architecture, architecture_of, get_architecture, known_architectures, load_config,
                       register_architecture, unregister_architecture)

__all__ = ["ConfigError", "ModelConfig", "key", "EngineOptions", "Architecture", "architecture_of",
           "get_architecture", "known_architectures", "load_config", "register_architecture",
           "unregister_architecture"]
