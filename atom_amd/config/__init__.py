from .engine_config import Config
from .model_config import ConfigError, ModelConfig, Qwen3Config, read_config_json
from .registry import (Architecture, build_model, get_architecture, known_architectures, model_config_from_dict,
                       register_architecture, unregister_architecture)

__all__ = ["Config", "ConfigError", "ModelConfig", "Qwen3Config", "read_config_json", "Architecture", "build_model",
           "get_architecture", "known_architectures", "model_config_from_dict", "register_architecture",
           "unregister_architecture"]
