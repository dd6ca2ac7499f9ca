from .base import (ConfigError, ModelConfig, architecture_of, config_from_dict, config_from_dir,
                   known_architectures, lookup, register_architecture)
from .llama import LlamaConfig

__all__ = ["ConfigError", "ModelConfig", "LlamaConfig", "architecture_of", "config_from_dict",
           "config_from_dir", "known_architectures", "lookup", "register_architecture"]
