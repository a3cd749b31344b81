from .base import ConfigError, ModelConfig, read_config_json
from .registry import (Architecture, architecture_name, get_architecture, load_config,
                       register_architecture, registered_architectures)
from .qwen2 import Qwen2Config

__all__ = ["ConfigError", "ModelConfig", "read_config_json", "Architecture", "architecture_name",
           "get_architecture", "load_config", "register_architecture", "registered_architectures",
           "Qwen2Config"]
