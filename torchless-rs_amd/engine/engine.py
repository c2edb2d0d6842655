"""The step function: a batch of sequences, their new tokens, logits back.

The reference forwards one token of one sequence per call and feeds a prompt
by calling that once per token (src/model/mod.rs:430-447,
src/main.rs:557-563); its batch sketch only keeps books
(src/model/batching.rs:585-614).  Here one `step` takes, for each sequence of
a batch, the tokens it brings (a whole prompt, or one decoded token, or any
number in between), runs exactly those rows from the cache that earlier
steps left, commits their keys and values, and returns float32 logits at
the rows asked for.  A sequence's result does not depend on its batch-mates.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.cache import PAGE, Cache
from ..config.base import ModelConfig, load_config
from ..parts.base import StepContext, Workspace
from ..weights.safetensors_io import ModelFiles, TensorDict
from .model import Model


class StepError(ValueError):
    """A step that cannot be run as asked (unknown slot, token id outside the
    vocabulary, empty batch, ...)."""


@dataclass
class SeqInput:
    """What one sequence brings to a step."""
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()          # indices among `tokens` whose logits are wanted


def resolve_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        return name
    table = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
             "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}
    if name not in table:
        raise ValueError(f"dtype {name!r} is not served; use one of {sorted(table)}")
    return table[name]


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError(f"the engine runs on the GPU only (asked for {device}); there is no CPU path")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to torch; the engine has no CPU path")
    return device


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0") -> Model:
    """A model from a folder with config.json and safetensors; the class of
    the configuration and the parts follow from config.json's architecture."""
    from ..models import model_spec_for
    from ..kernels.build import load as load_kernels
    device = require_gpu(device)
    load_kernels()                                   # fail here, loudly, if it cannot be had
    cfg = load_config(model_dir)
    model = Model(model_spec_for(cfg), cfg, resolve_dtype(dtype), device)
    model.load_weights(ModelFiles(model_dir))
    return model


def model_from_tensors(config: ModelConfig, tensors: Dict[str, torch.Tensor], dtype="bfloat16",
                       device="cuda:0") -> Model:
    from ..models import model_spec_for
    from ..kernels.build import load as load_kernels
    device = require_gpu(device)
    load_kernels()
    model = Model(model_spec_for(config), config, resolve_dtype(dtype), device)
    model.load_weights(TensorDict(tensors))
    return model


def build_context(cache: Cache, batch: Sequence[SeqInput], vocab_size: int, dtype: torch.dtype, device,
                  workspace: Workspace) -> Tuple[StepContext, Optional[torch.Tensor], int]:
    """Check a step's entries, get their pages, and lay the batch out on the
    device: tokens, row positions, row-to-sequence map, prefix sums, lengths and
    page tables in one upload.  Returns the context, the wanted rows (device,
    int32) and their number."""
    if not batch:
        raise StepError("a step needs at least one sequence")
    B = len(batch)
    n_new = np.zeros(B, dtype=np.int64)
    for b, s in enumerate(batch):
        if not cache.slots.holds(s.slot):
            raise StepError(f"entry {b}: slot {s.slot} is not held")
        n_new[b] = len(s.tokens)
        if n_new[b] < 1:
            raise StepError(f"entry {b}: a sequence must bring at least one token")
        for w in s.want:
            if not (0 <= w < n_new[b]):
                raise StepError(f"entry {b}: wanted index {w} outside its {n_new[b]} tokens")
    N = int(n_new.sum())
    tokens = np.concatenate([np.asarray(s.tokens, dtype=np.int64) for s in batch])
    if tokens.min() < 0 or tokens.max() >= vocab_size:
        bad = int(tokens[(tokens < 0) | (tokens >= vocab_size)][0])
        raise StepError(f"token id {bad} is outside the vocabulary of {vocab_size}")
    growth = [(s.slot, int(n)) for s, n in zip(batch, n_new)]
    len_before = np.array([cache.length[s.slot] for s in batch], dtype=np.int64)
    cache.prepare(growth)                       # raises CacheFull / CacheMisuse untouched
    len_after = len_before + n_new
    cu = np.zeros(B + 1, dtype=np.int64)
    np.cumsum(n_new, out=cu[1:])
    row_seq = np.repeat(np.arange(B), n_new)
    row_pos = np.arange(N) - cu[row_seq] + len_before[row_seq]
    want_rows = np.array([cu[b] + w for b, s in enumerate(batch) for w in s.want], dtype=np.int64)
    tables = []
    for g in cache.groups:
        stride = max(1, max(len(g.pages_of_slot[s.slot]) for s in batch))
        t = np.zeros((B, stride), dtype=np.int64)
        for b, s in enumerate(batch):
            pg = g.pages_of_slot[s.slot]
            t[b, :len(pg)] = pg
        tables.append(t)
    # one upload for all of it
    parts = [tokens, row_pos, row_seq, cu, np.array([s.slot for s in batch]), len_before,
             len_after, want_rows] + [t.reshape(-1) for t in tables]
    flat = np.concatenate(parts).astype(np.int32)
    dev = torch.from_numpy(flat).to(device, non_blocking=False)
    views, off = [], 0
    for p in parts:
        views.append(dev[off:off + p.size])
        off += p.size
    ctx = StepContext(
        n_rows=N, n_seqs=B, dtype=dtype, device=device,
        tokens=views[0], row_pos=views[1], row_seq=views[2], cu_seqlens=views[3], slots=views[4],
        len_before=views[5], len_after=views[6],
        tables={gi: views[8 + gi].view(B, tables[gi].shape[1]) for gi in range(len(tables))},
        all_single=bool((n_new == 1).all()), max_new=int(n_new.max()),
        max_len_after=int(len_after.max()), workspace=workspace, cache=cache,
        host={"n_new": n_new, "len_before": len_before, "len_after": len_after, "cu": cu,
              "slots": [s.slot for s in batch]})
    return ctx, (views[7] if want_rows.size else None), int(want_rows.size)



class Engine:
    """A model, its cache and workspace.  `max_tokens` is the most positions
    that live sequences hold at any time, each rounded up to whole pages."""

    def __init__(self, model: Model, max_tokens: int, max_slots: Optional[int] = None):
        self.model = model
        self.device = model.device
        self.cache: Cache = model.make_cache(max_tokens, max_slots)
        self.runs = model.bind_cache(self.cache)
        self.workspace = Workspace(self.device)
        self.vocab_size = model.spec.vocab_size

    # ---- slots -----------------------------------------------------------
    def alloc(self) -> int:
        return self.cache.alloc_slot()

    def free(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length[slot]

    def fits(self, lengths: List[int]) -> bool:
        """Can new sequences that grow to these lengths be held now?"""
        return self.cache.fits(list(lengths))

    # ---- the step ----------------------------------------------------------
    def build_context(self, batch: Sequence[SeqInput]) -> Tuple[StepContext, Optional[torch.Tensor], int]:
        return build_context(self.cache, batch, self.vocab_size, self.model.dtype, self.device,
                             self.workspace)

    def step(self, batch: Sequence[SeqInput]) -> torch.Tensor:
        """Run one step; returns float32 logits [number of wanted rows, V] in
        the order of the entries and of their `want` lists.  The tensor is a
        view of the engine's workspace: it is overwritten by the next step."""
        ctx, want_rows, n_want = self.build_context(batch)
        logits = self.model.forward(ctx, self.runs, want_rows, n_want)
        self.cache.commit([(s.slot, len(s.tokens)) for s in batch])
        return logits
