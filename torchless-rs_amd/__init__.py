"""A small MI355X-native model library with generation: configuration and
registry, weights by name, parts, a paged cache, one step function, a
generation loop with sampling, and the HIP kernels under them."""
from . import models as _models                      # registers the architectures
from .config import (ConfigError, MistralConfig, ModelConfig, config_from_dict, load_config,
                     register_architecture, registered_architectures)
from .sampling.config import SamplingConfig
from .weights import WeightBindingError, write_random_model

__all__ = ["ConfigError", "MistralConfig", "ModelConfig", "config_from_dict", "load_config",
           "register_architecture", "registered_architectures", "WeightBindingError",
           "write_random_model", "SamplingConfig", "Engine", "SeqInput", "load_model",
           "model_from_tensors", "generate", "generate_until_eos", "GenerationResult"]

_LAZY = {"Engine": "engine.engine", "SeqInput": "engine.engine", "load_model": "engine.engine",
         "model_from_tensors": "engine.engine", "generate": "api", "generate_until_eos": "api",
         "GenerationResult": "engine.generate"}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        return getattr(importlib.import_module("." + _LAZY[name], __name__), name)
    raise AttributeError(name)
