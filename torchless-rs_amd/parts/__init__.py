from .base import (FeedForward, LayerSpec, Mixer, ModelSpec, Norm, Part, PartSpec, Position, Run,
                   RunBinding, StepContext, Workspace, make_part, register_part, registered_parts,
                   unregister_part)
from . import attention, block, embedding, ffn, norms, position   # noqa: F401  (register)
from .linear import Linear

__all__ = ["FeedForward", "LayerSpec", "Linear", "Mixer", "ModelSpec", "Norm", "Part", "PartSpec",
           "Position", "Run", "RunBinding", "StepContext", "Workspace", "make_part",
           "register_part", "registered_parts", "unregister_part"]
