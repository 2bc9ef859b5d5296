from .fields import ConfigError
from .qwen2 import Qwen2Config
from .registry import (Architecture, architecture_named, architecture_of, load_config,
                       register_architecture, registered_architectures, unregister_architecture)

__all__ = ["ConfigError", "Qwen2Config", "Architecture", "architecture_named", "architecture_of",
           "load_config", "register_architecture", "registered_architectures", "unregister_architecture"]
