from .base import (ArchitectureEntry, ConfigError, ModelConfig, architecture_name,
                   config_from_dict, get_architecture, load_config, register_architecture,
                   registered_architectures, unregister_architecture)
from .mistral import MistralConfig

__all__ = ["ArchitectureEntry", "ConfigError", "ModelConfig", "MistralConfig", "architecture_name",
           "config_from_dict", "get_architecture", "load_config", "register_architecture",
           "registered_architectures", "unregister_architecture"]
