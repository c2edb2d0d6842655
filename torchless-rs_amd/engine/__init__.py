from .engine import (Engine, SeqInput, StepError, load_model, model_from_tensors, require_gpu,
                     resolve_dtype)
from .model import Model

__all__ = ["Engine", "Model", "SeqInput", "StepError", "load_model", "model_from_tensors",
           "require_gpu", "resolve_dtype"]
