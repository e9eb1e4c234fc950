from .model_config import ConfigError, Qwen3Config, parse_eos_token_ids, read_config_json
from .registry import (Architecture, UnknownArchitecture, register_architecture, registered_architectures,
                       resolve_architecture)
from .engine_config import EngineConfig

__all__ = ["ConfigError", "Qwen3Config", "parse_eos_token_ids", "read_config_json", "Architecture",
           "UnknownArchitecture", "register_architecture", "registered_architectures", "resolve_architecture",
           "EngineConfig"]
