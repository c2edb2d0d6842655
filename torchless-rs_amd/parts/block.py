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

    def entry_norm(self):
        """The norm that reads the stream first, if the part behind it can take a norm cut in
        two (the block before this one may then do the norm's first half)."""
        ok = self.mixer_norm.rms_form() is not None and getattr(self.mixer, "takes_row_factor", False)
        return self.mixer_norm if ok else None

    def forward(self, ctx, run, x: torch.Tensor, norm_after=None) -> None:
        """`norm_after`: the `entry_norm` of the block that runs next, if it has one."""
        y = ctx.workspace.get("block_y", tuple(x.shape), ctx.dtype)
        y1 = self._norm(self.mixer_norm, ctx, x, y)
        if (self.ffn_norm.rms_form() is not None and getattr(self.ffn, "takes_row_factor", False)
                and getattr(self.mixer, "closes_stream", False)):
            ctx.norm_ahead = self.ffn_norm
        self.mixer.forward(ctx, run, y1, x)
        self._after_part(ctx, self.mixer)
        y2 = self._norm(self.ffn_norm, ctx, x, y)
        if getattr(self.ffn, "closes_stream", False):
            ctx.norm_ahead = norm_after
        self.ffn.forward(ctx, y2, x)
        self._after_part(ctx, self.ffn)

    @staticmethod
    def _after_part(ctx, part) -> None:
        ctx.norm_ahead = None
        if ctx.row_factor is not None:
            raise RuntimeError(f"{type(part).__name__} declares takes_row_factor and left the factor untaken")

    @staticmethod
    def _norm(norm, ctx, x, y) -> torch.Tensor:
        """A norm reads the stream: partial products that a part left pending are
        added first, by the norm itself if it can (`takes_pending`).  If the product
        that completed the stream did this norm's first half, the output is what it
        left, and the factor per row goes to the part that reads it."""
        pre, ctx.prenormed = ctx.prenormed, None
        if pre is not None and pre[0] is norm:
            ctx.row_factor = pre[2]
            ctx.settle = lambda: norm.forward(ctx, x, pre[1])      # the plain norm into the same buffer
            return pre[1]
        if not getattr(norm, "takes_pending", False):
            flush_pending(ctx, x)
        norm.forward(ctx, x, y)
        return y


register_part("block", "pre_norm", PreNormBlock)
