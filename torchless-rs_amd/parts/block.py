"""The arrangement of a layer: x += mixer(norm(x)); x += ffn(norm(x))
(src/model/modules/layer.rs:28-56 of the reference).  The residual stream x
is float32; mixer and feed-forward add into it."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.binding import WeightSpec
from .base import LayerSpec, Part, flush_pending, make_part, register_part


class PreNormBlock(Part):
    def __init__(self, layer: LayerSpec, mixer_norm_name: str = "input_layernorm.",
                 ffn_norm_name: str = "post_attention_layernorm."):
        self.mixer = make_part("mixer", layer.mixer)
        self.ffn = make_part("ffn", layer.ffn)
        self.mixer_norm = make_part("norm", layer.mixer_norm)
        self.ffn_norm = make_part("norm", layer.ffn_norm)
        self.n1, self.n2 = mixer_norm_name, ffn_norm_name
        self.graph_safe = all(p.graph_safe for p in (self.mixer, self.ffn, self.mixer_norm, self.ffn_norm))

    def weight_specs(self) -> Dict[str, WeightSpec]:
        out: Dict[str, WeightSpec] = {}
        for k, v in self.mixer_norm.weight_specs().items():
            out[self.n1 + k] = v
        out.update(self.mixer.weight_specs())
        for k, v in self.ffn_norm.weight_specs().items():
            out[self.n2 + k] = v
        out.update(self.ffn.weight_specs())
        return out

    def load(self, tensors, compute_dtype) -> None:
        def sub(prefix):
            return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}
        self.mixer_norm.load(sub(self.n1), compute_dtype)
        self.ffn_norm.load(sub(self.n2), compute_dtype)
        self.mixer.load(tensors, compute_dtype)
        self.ffn.load(tensors, compute_dtype)

    def forward(self, ctx, run, x: torch.Tensor) -> None:
        y = ctx.workspace.get("block_y", tuple(x.shape), ctx.dtype)
        self._norm(self.mixer_norm, ctx, x, y)
        self.mixer.forward(ctx, run, y, x)
        self._norm(self.ffn_norm, ctx, x, y)
        self.ffn.forward(ctx, y, x)

    @staticmethod
    def _norm(norm, ctx, x, y) -> None:
        """A norm reads the stream: partial products that a part left pending are
        added first, by the norm itself if it can (`takes_pending`)."""
        if not getattr(norm, "takes_pending", False):
            flush_pending(ctx, x)
        norm.forward(ctx, x, y)


register_part("block", "pre_norm", PreNormBlock)
