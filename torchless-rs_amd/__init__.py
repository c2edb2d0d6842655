"""A small MI355X-native model library with generation: configuration and
registry, weights by name, parts, a paged cache, one step function, a
generation loop with sampling, and the HIP kernels under them."""
from . import models as _models                      # registers the architectures
from .config import (ConfigError, MistralConfig, ModelConfig, config_from_dict, load_config,
                     register_architecture, registered_architectures)
from .weights import WeightBindingError, write_random_model

__all__ = ["ConfigError", "MistralConfig", "ModelConfig", "config_from_dict", "load_config",
           "register_architecture", "registered_architectures", "WeightBindingError",
           "write_random_model"]
