"""Rotary position encoding.

inv_freq[i] = 1 / theta^(i / (r/2)) for the r rotated channels of a head; pair i
is rotated by the angle pos * inv_freq[i].  The reference rotates the whole head
(r = d) in pairs (i, i + d/2) (src/kernels/mod.rs:572-608); `rotary_dim` < d
rotates the first channels only and `interleaved` pairs (2i, 2i+1) instead.
Angles, cosines and sines are float32.  The table of inverse frequencies is made
once on the host in float64 and rounded to float32.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Position, register_part


class Rotary(Position):
    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None, interleaved: bool = False):
        self.head_dim = int(head_dim)
        self.rotary_dim = self.head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rotary: {self.rotary_dim} rotated channels of a head of {self.head_dim} "
                             "(even, at most the head)")
        self.theta = float(theta)
        self.interleaved = bool(interleaved)
        self._rotation = {}

    def inv_freq_host(self) -> torch.Tensor:
        half = self.rotary_dim // 2
        i = torch.arange(half, dtype=torch.float64)
        return (1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64), i / half)).to(torch.float32)

    def rotation(self, device) -> ops.Rotation:
        key = str(device)
        if key not in self._rotation:
            self._rotation[key] = ops.Rotation(self.inv_freq_host().to(device), self.rotary_dim, self.interleaved)
        return self._rotation[key]

    def inv_freq(self, device) -> torch.Tensor:
        """The frequencies alone (float32 [rotary_dim / 2] on `device`)."""
        return self.rotation(device).inv_freq


class NoPosition(Position):
    """Queries and keys are used as they are (the base class's answer)."""

    def __init__(self, head_dim: int = 0):
        self.head_dim = int(head_dim)


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
