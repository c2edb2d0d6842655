"""Rotary position encoding, half-split pairing.

inv_freq[i] = 1 / theta^(i / (d/2)); the pair (i, i + d/2) of a head is
rotated by the angle pos * inv_freq[i] (src/kernels/mod.rs:572-608 of the
reference).  Angles, cosines and sines are float32.  The table of inverse
frequencies is made once on the host in float64 and rounded to float32.
"""
from __future__ import annotations

import torch

from .base import Position, register_part


class Rotary(Position):
    def __init__(self, head_dim: int, theta: float):
        if head_dim % 2:
            raise ValueError(f"rotary: head_dim {head_dim} must be even")
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self._inv_freq = {}

    def inv_freq_host(self) -> torch.Tensor:
        half = self.head_dim // 2
        i = torch.arange(half, dtype=torch.float64)
        return (1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64), i / half)).to(torch.float32)

    def inv_freq(self, device) -> torch.Tensor:
        key = str(device)
        if key not in self._inv_freq:
            self._inv_freq[key] = self.inv_freq_host().to(device)
        return self._inv_freq[key]


register_part("position", "rotary", Rotary)
