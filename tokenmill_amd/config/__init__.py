from tokenmill_amd.config.engine_config import EngineConfig, add_engine_args, engine_config_from_args
from tokenmill_amd.config.model_config import ConfigError, Qwen2Config
from tokenmill_amd.config.registry import (Architecture, get_architecture, known_architectures, load_config,
                                           register_architecture)

__all__ = ["EngineConfig", "add_engine_args", "engine_config_from_args", "ConfigError", "Qwen2Config",
           "Architecture", "get_architecture", "known_architectures", "load_config", "register_architecture"]
