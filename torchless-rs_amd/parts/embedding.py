"""Token embedding (a row copy, no scaling: src/model/modules/embedding.rs:15-21
of the reference) and the output head (logits = W x, its own tensor unless the
configuration ties it to the embedding: src/model/mod.rs:364-369, 443-446)."""
from __future__ import annotations

from typing import Dict

import torch

from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Part, register_part
from .linear import Linear


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, name: str = "embed_tokens.weight"):
        self.V, self.H, self.name = int(vocab_size), int(hidden_size), name
        self.table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.V, self.H))}

    def load(self, tensors, compute_dtype) -> None:
        self.table = tensors[self.name]

    def forward(self, ctx, ids: torch.Tensor, x: torch.Tensor) -> None:
        ops.embed(self.table, ids, x)


class LMHead(Part):
    """`tied`: use the embedding table instead of a tensor of its own."""
    graph_safe = True

    def may_capture(self, n_rows: int) -> bool:
        return self.proj is not None and self.proj.own_kernels(n_rows)

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, name: str = "weight"):
        self.V, self.H, self.tied, self.name = int(vocab_size), int(hidden_size), bool(tied), name
        self.proj = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {} if self.tied else {self.name: WeightSpec((self.V, self.H))}

    def load(self, tensors, compute_dtype) -> None:
        self.proj = Linear(tensors["__embedding__"] if self.tied else tensors[self.name])

    def forward(self, ctx, y: torch.Tensor, logits: torch.Tensor) -> None:
        self.proj(y, logits)


register_part("embedding", "tokens", TokenEmbedding)
register_part("head", "linear", LMHead)
