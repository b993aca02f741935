from .errors import ConfigError
from .qwen3 import Qwen3Config
from .registry import (Architecture, register_architecture, resolve_architecture, known_architectures,
                       load_config, read_config_json)

__all__ = ["ConfigError", "Qwen3Config", "Architecture", "register_architecture", "resolve_architecture",
           "known_architectures", "load_config", "read_config_json"]
