"""Architectures: each module registers a name from config.json's
`architectures` with its configuration class and its `ModelSpec` builder."""
from ..config.base import ModelConfig, get_architecture
from ..parts import base as _parts_base
from .. import parts as _parts            # registers the parts
from . import mistral as _mistral         # registers MistralForCausalLM


def model_spec_for(cfg: ModelConfig):
    return get_architecture(cfg.architecture).build_spec(cfg)
