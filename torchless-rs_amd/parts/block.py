"""The arrangement of a layer: x += mixer(norm(x)); x += ffn(norm(x))
(src/model/modules/layer.rs:28-56 of the reference).  The residual stream x
is float32; mixer and feed-forward add into it."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.binding import WeightSpec
from .base import (LayerSpec, Part, expect_norm, make_part, part_done, read_through_norm, register_part,
                   splittable_entry)


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

    def may_capture(self, n_rows: int) -> bool:
        return all(p.may_capture(n_rows) for p in (self.mixer, self.ffn, self.mixer_norm, self.ffn_norm))

    def prefers_eager(self, n_new, len_before, device) -> bool:
        return any(p.prefers_eager(n_new, len_before, device) for p in (self.mixer, self.ffn, self.mixer_norm, self.ffn_norm))

    def entry_norm(self):
        """The norm that reads the stream first, if the part behind it can take a norm cut in
        two (the block before this one may then do the norm's first half)."""
        return splittable_entry(self.mixer_norm, self.mixer)

    def forward(self, ctx, run, x: torch.Tensor, norm_after=None) -> None:
        """`norm_after`: the `entry_norm` of the block that runs next, if it has one.  The three
        helpers around each part (`read_through_norm`, `expect_norm`, `part_done`) are all that
        an arrangement needs for norms cut in two around the products."""
        y = ctx.workspace.get("block_y", tuple(x.shape), ctx.dtype)
        y1 = read_through_norm(ctx, self.mixer_norm, x, y)
        expect_norm(ctx, self.mixer, self.ffn_norm, self.ffn)
        self.mixer.forward(ctx, run, y1, x)
        part_done(ctx, self.mixer)
        y2 = read_through_norm(ctx, self.ffn_norm, x, y)
        expect_norm(ctx, self.ffn, norm_after)
        self.ffn.forward(ctx, y2, x)
        part_done(ctx, self.ffn)


register_part("block", "pre_norm", PreNormBlock)
