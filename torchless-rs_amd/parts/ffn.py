"""SwiGLU feed-forward: down( silu(gate y) * (up y) ), silu(g) = g / (1 + e^-g)
(src/model/modules/mlp.rs:23-45, src/kernels/mod.rs:546-548 of the reference).
gate and up are bound under their own names (`names`: the leaf names are
parameters, and a checkpoint that stores gate|up as one tensor binds that one)
and laid side by side at load so that one product serves both."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import FeedForward, register_part, take_row_factor
from .linear import Linear, interleave_pairs


class SwiGLU(FeedForward):
    graph_safe = True
    closes_stream = True          # its last write to the stream is `Linear.add_into`
    takes_row_factor = True       # its gate|up product can do the division of the norm before it

    # leaf names of the tensors under `prefix`; "gate_up": one tensor [gate | up] by rows instead of the two
    NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight", "gate_up": None}

    def __init__(self, hidden_size: int, intermediate_size: int, prefix: str = "mlp.",
                 names: Optional[Dict[str, Optional[str]]] = None):
        self.H = int(hidden_size)
        self.I = int(intermediate_size)
        self.prefix = prefix
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"swiglu: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        self.gate_up = None
        self.down = None

    def may_capture(self, n_rows: int) -> bool:
        return self.gate_up is not None and self.gate_up.own_kernels(n_rows) and self.down.own_kernels(n_rows)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        if nm["gate_up"]:
            return {p + nm["gate_up"]: WeightSpec((2 * self.I, self.H)), p + nm["down"]: WeightSpec((self.H, self.I))}
        return {p + nm["gate"]: WeightSpec((self.I, self.H)),
                p + nm["up"]: WeightSpec((self.I, self.H)),
                p + nm["down"]: WeightSpec((self.H, self.I))}

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names
        if nm["gate_up"]:
            g, u = tensors[p + nm["gate_up"]][:self.I], tensors[p + nm["gate_up"]][self.I:]
        else:
            g, u = tensors[p + nm["gate"]], tensors[p + nm["up"]]
        if g.dtype != u.dtype:
            g, u = g.to(torch.float32), u.to(torch.float32)
        # bfloat16 on the matrix cores: gate and up rows interleaved so that the product's
        # epilogue applies silu(gate) * up itself and writes bfloat16
        self.paired = (compute_dtype == torch.bfloat16 and g.dtype == torch.bfloat16 and self.I % 32 == 0
                       and self.H % 8 == 0)
        self.gate_up = Linear(interleave_pairs(g, u) if self.paired else torch.cat([g, u], dim=0))
        self.down = Linear(tensors[p + nm["down"]], tiled=True)

    def forward(self, ctx, y: torch.Tensor, x: torch.Tensor) -> None:
        n = y.shape[0]
        h = ctx.workspace.get("ffn_h", (n, self.I), ctx.dtype)
        factor = take_row_factor(ctx, usable=self.paired and ops.norm_split_ok(y, self.gate_up.weight))
        if factor is not None:
            ops.gemm_bf16_norm(y, self.gate_up.weight, h, silu_pair=True, factor=factor)
        elif self.paired and self.gate_up.mid(y):
            ops.gemm_mid_bf16(y, self.gate_up.weight, h, 1, silu_pair=True)
        elif self.paired and ops.bf16_gemm_ok(y, self.gate_up.weight):
            if n > ops.LIBRARY_ROWS:
                gu = ctx.workspace.get("ffn_gu16", (n, 2 * self.I), torch.bfloat16)
                ops.gemm_library(y, self.gate_up.weight, gu)
                ops.silu_mul_pairs(gu, h)
            else:
                ops.gemm_bf16(y, self.gate_up.weight, h, silu_pair=True)
        else:
            gu = ctx.workspace.get("ffn_gu", (n, 2 * self.I), torch.float32)
            self.gate_up(y, gu)
            ops.silu_mul(gu, h)
        self.down.add_into(h, x, ctx, "ffn_down_parts")


register_part("ffn", "swiglu", SwiGLU)
