"""Options of sampling, with the reference's names and meanings
(src/sampler/mod.rs:17-54): temperature 0 is greedy, 1 leaves the logits as
they are; top_k keeps the k largest logits; top_p keeps the smallest set of
tokens whose probability reaches p.  Order: temperature, top-k, softmax,
top-p, draw.  `seed` is ours: the reference draws from an unseeded generator
(src/sampler/mod.rs:226)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class SamplingConfig:
    temperature: float = 1.0
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    seed: int = 0

    @classmethod
    def greedy(cls) -> "SamplingConfig":
        return cls(temperature=0.0)

    @classmethod
    def with_temperature(cls, temperature: float, seed: int = 0) -> "SamplingConfig":
        return cls(temperature=temperature, seed=seed)

    @property
    def is_greedy(self) -> bool:
        return not self.temperature > 0.0
