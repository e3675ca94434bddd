from .engine_config import EngineConfig
from .model_config import ConfigError, LlamaConfig, ModelConfig, read_config_json
from .registry import (Architecture, architecture_for, architecture_of, known_architectures, known_shapes,
                       load_model_config, shape_config, register_architecture, unregister_architecture)

__all__ = ["EngineConfig", "ConfigError", "LlamaConfig", "ModelConfig", "read_config_json", "Architecture",
           "architecture_for", "architecture_of", "known_architectures", "known_shapes", "shape_config", "load_model_config",
           "register_architecture", "unregister_architecture"]
