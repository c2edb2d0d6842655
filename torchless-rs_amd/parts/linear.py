"""Products with a weight matrix stored [out, in] as the checkpoint has it
(out[r] = sum_c W[r,c] x[c], src/loader/parameters.rs:551-594 of the
reference).  The kernel is chosen by what the operands are, never by the
model: float32 anywhere means the plain FMA kernel (true 32-bit)."""
from __future__ import annotations

import torch

from ..kernels import ops


class Linear:
    """A weight [N, K] resident on the device in its stored width."""

    def __init__(self, weight: torch.Tensor):
        assert weight.dim() == 2
        self.weight = weight.contiguous()
        self.out_features, self.in_features = self.weight.shape

    def __call__(self, a: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
        """out[M, N] (+)= a[M, K] @ W^T; out is float32."""
        ops.gemm(a, self.weight, out, accumulate)


def interleave_pairs(gate: torch.Tensor, up: torch.Tensor, block: int = 32) -> torch.Tensor:
    """Rows in groups of 2*block: `block` rows of gate, then the `block` rows of
    up that belong to them: the layout of the products' paired epilogue."""
    I, K = gate.shape
    g = gate.view(I // block, block, K)
    u = up.view(I // block, block, K)
    return torch.stack([g, u], dim=1).reshape(2 * I, K).contiguous()
