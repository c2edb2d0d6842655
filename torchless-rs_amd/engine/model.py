"""A model put together from a `ModelSpec`: parts built, weights bound, runs of
the schedule tied to their places in the cache.

The reference's `Mistral::load` binds tensors by hard-coded names and its
`forward` walks embedding, layers, norm and head for one token
(src/model/mod.rs:354-447).  Here the same walk goes over the rows of a whole
step, and which parts it meets is data.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.cache import Cache, KVRequest, StateRequest
from ..config.base import ModelConfig
from ..parts.base import ModelSpec, PartSpec, RunBinding, StepContext, flush_pending, make_part
from ..weights.binding import bind_weights


class Model:
    def __init__(self, spec: ModelSpec, config: Optional[ModelConfig], dtype: torch.dtype, device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
        self.spec = spec
        self.config = config
        self.dtype = dtype
        self.device = torch.device(device)
        self.embedding = make_part("embedding", spec.embedding)
        self.blocks = [make_part("block", PartSpec(ls.block.kind, dict(ls.block.params, layer=ls)))
                       for ls in spec.layers]
        self.final_norm = make_part("norm", spec.final_norm)
        self.head = make_part("head", spec.head)
        for i, run in enumerate(spec.schedule):
            if not (0 <= run.layer < len(self.blocks)):
                raise ValueError(f"schedule entry {i} names layer {run.layer}, there are "
                                 f"{len(self.blocks)}")
            if run.kv_from is not None and not (0 <= run.kv_from < i):
                raise ValueError(f"schedule entry {i} reads the cache of entry {run.kv_from}, which "
                                 "is not an earlier one")
        self.loaded = False
        self.graph_safe = all(p.graph_safe for p in [self.embedding, self.final_norm, self.head] + self.blocks)

    def may_capture(self, n_rows: int) -> bool:
        """May a single-token step of `n_rows` rows be captured as a graph and replayed?  Every
        part answers for itself; the step function knows nothing of their kernels."""
        return self.loaded and all(p.may_capture(n_rows)
                                   for p in [self.embedding, self.final_norm, self.head] + self.blocks)

    def prefers_eager(self, n_new, len_before, device) -> bool:
        """Does any part want to shape its launches by this step's own lengths (see `Part.prefers_eager`)?"""
        return any(p.prefers_eager(n_new, len_before, device)
                   for p in [self.embedding, self.final_norm, self.head] + self.blocks)

    # ---- weights -----------------------------------------------------------
    def load_weights(self, source, tiled_copies: bool = True) -> None:
        """`source`: anything with names/shape/dtype/tensor (a model folder's
        files, or tensors in memory).  `tiled_copies`: may the parts keep second
        copies of weights in the layout that single-token steps stream fastest?"""
        from ..parts.linear import loading_with
        with loading_with(tiled_copies):
            self._load_parts(source)

    def _load_parts(self, source) -> None:
        spec = self.spec
        t = bind_weights(spec.weight_specs(), source, self.dtype, self.device, spec.ignore_tensors)

        def sub(prefix: str) -> Dict[str, torch.Tensor]:
            return {k[len(prefix):]: v for k, v in t.items() if k.startswith(prefix)}

        self.embedding.load(sub(spec.embedding_prefix), self.dtype)
        for ls, blk in zip(spec.layers, self.blocks):
            blk.load(sub(ls.prefix), self.dtype)
        self.final_norm.load(sub(spec.final_norm_prefix), self.dtype)
        head_t = sub(spec.head_prefix)
        head_t["__embedding__"] = getattr(self.embedding, "table", None)
        self.head.load(head_t, self.dtype)
        self.loaded = True

    # ---- cache ---------------------------------------------------------------
    def cache_requests(self):
        kv: Dict[int, KVRequest] = {}
        st: Dict[int, StateRequest] = {}
        for i, run in enumerate(self.spec.schedule):
            mixer = self.blocks[run.layer].mixer
            if run.kv_from is None:
                r = mixer.kv_request()
                if r is not None:
                    kv[i] = r
            s = mixer.state_request()
            if s is not None:
                st[i] = s
        return kv, st

    def make_cache(self, max_tokens: int, max_slots: Optional[int] = None, allocate: bool = True) -> Cache:
        kv, st = self.cache_requests()
        return Cache(kv, st, max_tokens, self.dtype, self.device, max_slots, allocate)

    def bind_cache(self, cache: Cache) -> List[RunBinding]:
        """Tie every run of the schedule to its place in `cache`."""
        read_later = {r.kv_from for r in self.spec.schedule if r.kv_from is not None}
        runs: List[RunBinding] = []
        for i, run in enumerate(self.spec.schedule):
            src = i if run.kv_from is None else run.kv_from
            b = RunBinding(index=i, kv_owner=run.kv_from is None, kv_source=src,
                           kv_read_later=i in read_later, state=cache.state.get(i))
            if src in cache.group_of_run:
                b.kv_group_index = cache.group_of_run[src]
                b.kv_group, b.kv_layer = cache.kv_layer(src)
            elif run.kv_from is not None:
                raise ValueError(f"schedule entry {i} reads the cache of entry {src}, which keeps none")
            runs.append(b)
        return runs

    # ---- one step ------------------------------------------------------------
    def forward(self, ctx: StepContext, runs: List[RunBinding], want_rows: Optional[torch.Tensor],
                n_want: int) -> torch.Tensor:
        """Run the rows of `ctx` through the schedule and return float32 logits
        [n_want, V] at `want_rows` (int32 row indices on the device)."""
        if not self.loaded:
            raise RuntimeError("the model has no weights yet")
        H, V = self.spec.hidden_size, self.spec.vocab_size
        ws = ctx.workspace
        x = ws.get("residual", (ctx.n_rows, H), torch.float32)
        self.embedding.forward(ctx, ctx.tokens, x)
        order = [self.blocks[run.layer] for run in self.spec.schedule]
        for i, (block, binding) in enumerate(zip(order, runs)):
            after = order[i + 1].entry_norm() if i + 1 < len(order) and hasattr(order[i + 1], "entry_norm") else None
            if after is not None:
                block.forward(ctx, binding, x, norm_after=after)
            else:
                block.forward(ctx, binding, x)
        ctx.prenormed = None                 # nothing reads a norm's first half past the last block
        for commit in ctx.host.pop("deferred", []):
            commit()
        flush_pending(ctx, x)
        logits = ws.get("logits", (n_want, V), torch.float32)
        if n_want:
            xs = ws.get("head_x", (n_want, H), torch.float32)
            from ..kernels import ops
            ops.gather_rows(x, want_rows, xs)
            y = ws.get("head_y", (n_want, H), ctx.dtype)
            self.final_norm.forward(ctx, xs, y)
            self.head.forward(ctx, y, logits)
        return logits
