from .base import ConfigError, ModelConfig, UnsupportedModelError, field, read_config_json
from .named_sizes import NAMED_SIZES, named_config, named_size
from .qwen3 import Qwen3Config
from .registry import (config_from_dict, load_config, register_architecture, registered_architectures,
                       resolve_architecture, unregister_architecture)

__all__ = ["ConfigError", "ModelConfig", "UnsupportedModelError", "field", "read_config_json", "Qwen3Config", "NAMED_SIZES", "named_config", "named_size",
           "config_from_dict", "load_config", "register_architecture", "registered_architectures",
           "resolve_architecture", "unregister_architecture"]
