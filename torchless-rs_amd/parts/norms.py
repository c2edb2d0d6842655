"""RMSNorm.  y = x / sqrt(mean(x^2) + eps) * w, in float32
(src/kernels/mod.rs:558-568 of the reference; weight used as it is)."""
from __future__ import annotations

from typing import Dict

import torch

from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Norm, RmsForm, register_part


class RMSNorm(Norm):
    graph_safe = True
    takes_pending = True        # adds partial products left in ctx.pending while it reads the stream

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.size,), init="ones")}

    def load(self, tensors, compute_dtype) -> None:
        self.weight = tensors["weight"].to(torch.float32).contiguous()

    def rms_form(self) -> RmsForm:
        return RmsForm(self.weight, self.size, self.eps)

    def forward(self, ctx, x: torch.Tensor, out: torch.Tensor) -> None:
        """Partial products waiting in `ctx.pending` are added to x on the way."""
        pend = getattr(ctx, "pending", None)
        if pend is not None and self.size % 4 == 0 and self.size <= 8192:
            ops.add_rmsnorm(x, pend, self.weight, self.eps, out)
            ctx.pending = None
            return
        if pend is not None:
            ops.add_partials(x, pend)
            ctx.pending = None
        ops.rmsnorm(x, self.weight, self.eps, out)


register_part("norm", "rmsnorm", RMSNorm)
