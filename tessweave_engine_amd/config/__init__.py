from .model_config import ConfigError
from .engine_config import EngineConfig
from .registry import (Architecture, architecture_for, build_model, config_from_dict,
                       read_model_config, register_architecture, registered_architectures,
                       unregister_architecture)

__all__ = ["ConfigError", "EngineConfig", "Architecture", "architecture_for",
           "build_model", "config_from_dict", "read_model_config", "register_architecture",
           "registered_architectures", "unregister_architecture"]
