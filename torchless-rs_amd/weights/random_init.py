"""Random weights from a configuration and a seed.

The reference's fixture generator draws every tensor, norms included, from an
unseeded normal distribution (tests/generate_test_model.py:89-110).  Here the
draw is seeded: matrices N(0, std), norm weights N(1, norm_std) (exactly 1.0
when norm_std is 0), in the order in which the model names its tensors, each
drawn in float32 and then rounded to the storage dtype.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional, Union

import torch

from ..config.base import ModelConfig, config_from_dict
from .binding import WeightSpec
from .safetensors_io import write_safetensors


def random_tensors(expected: Dict[str, WeightSpec], seed: int, std: float = 0.02,
                   norm_std: float = 0.0, dtype: torch.dtype = torch.bfloat16,
                   device: Union[str, torch.device] = "cpu") -> Dict[str, torch.Tensor]:
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out: Dict[str, torch.Tensor] = {}
    for name, spec in expected.items():
        if spec.integer:
            out[name] = torch.zeros(spec.shape, dtype=torch.int32, device=device)
        elif spec.init == "ones":
            t = torch.ones(spec.shape, dtype=torch.float32, device=device)
            if norm_std:
                t += norm_std * torch.randn(spec.shape, generator=gen, dtype=torch.float32,
                                            device=device)
            out[name] = t.to(dtype)
        else:
            t = torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device)
            out[name] = t.mul_(std).to(dtype)
    return out


def write_random_model(model_dir: str, config: Union[dict, ModelConfig], seed: int,
                       std: float = 0.02, norm_std: float = 0.0,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write `config.json` and `model.safetensors` of a randomly initialised
    model into `model_dir` and return the folder."""
    from ..models import model_spec_for          # late: models imports the parts

    cfg = config_from_dict(config) if isinstance(config, dict) else config
    expected = model_spec_for(cfg).weight_specs()
    tensors = random_tensors(expected, seed, std, norm_std, dtype)
    os.makedirs(model_dir, exist_ok=True)
    d = cfg.to_dict()
    d["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32",
                        torch.float16: "float16"}[dtype]
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(d, f, indent=2)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return model_dir
