from .base import (Architecture, ConfigError, KeyReader, ModelConfig, architecture_of, build_model,
                   config_from_dict, known_architectures, load_config, read_config_json,
                   register_architecture)
from .llama import LlamaConfig, RopeScaling

__all__ = ["Architecture", "ConfigError", "KeyReader", "ModelConfig", "architecture_of", "build_model",
           "config_from_dict", "known_architectures", "load_config", "read_config_json",
           "register_architecture", "LlamaConfig", "RopeScaling"]
