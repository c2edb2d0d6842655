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

import ctypes
import gc
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.cache import PAGE, Cache
from ..config.base import ModelConfig, load_config
from ..parts.base import StepContext, Workspace
from ..weights.safetensors_io import ModelFiles, TensorDict
from .model import Model


from ..cache.native import StepError        # noqa: E402  (raised by the host library's packer too)


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


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0", tiled_copies: bool = True) -> Model:
    """A model from a folder with config.json and safetensors; the class of
    the configuration and the parts follow from config.json's architecture.
    `tiled_copies`: see `Model.load_weights`."""
    from ..models import model_spec_for
    from ..kernels.build import load as load_kernels
    device = require_gpu(device)
    load_kernels()                                   # fail here, loudly, if it cannot be had
    cfg = load_config(model_dir)
    model = Model(model_spec_for(cfg), cfg, resolve_dtype(dtype), device)
    model.load_weights(ModelFiles(model_dir), tiled_copies)
    return model


def model_from_tensors(config: ModelConfig, tensors: Dict[str, torch.Tensor], dtype="bfloat16",
                       device="cuda:0", tiled_copies: bool = True) -> Model:
    from ..models import model_spec_for
    from ..kernels.build import load as load_kernels
    device = require_gpu(device)
    load_kernels()
    model = Model(model_spec_for(config), config, resolve_dtype(dtype), device)
    model.load_weights(TensorDict(tensors), tiled_copies)
    return model


@dataclass
class PackedStep:
    """A step's batch on the host: one int32 array and where its pieces lie."""
    flat: np.ndarray
    sizes: List[int]                 # lengths of the pieces, in the order of `context_from`
    n_rows: int
    n_seqs: int
    n_want: int
    strides: Tuple[int, ...]         # page-table width of each cache group
    all_single: bool
    max_new: int
    max_len_after: int
    host: Dict[str, object]

    @property
    def key(self):
        """What a captured step of this shape must have in common with this one: every number that
        reaches a kernel from the host (sizes, page-table widths and, where sequences bring several
        tokens, how many each and the width of the buffers laid out by `aligned_columns`);
        everything else the kernels read on the device."""
        if self.all_single:
            return (self.n_seqs, self.n_rows, self.n_want, self.strides)
        return (self.n_seqs, self.n_rows, self.n_want, self.strides, tuple(int(n) for n in self.host["n_new"]),
                int(self.host["aligned_cols"]))


def pack_step(cache: Cache, batch: Sequence[SeqInput], vocab_size: int,
              token_rows: Optional[Sequence[int]] = None) -> PackedStep:
    """Check a step's entries, get their pages, and lay the batch out: tokens,
    row positions, row-to-sequence map, prefix sums, slots, lengths, wanted
    rows, aligned column offsets and page tables in one array (the work is the
    host library's `tl_pack_step`).  A page table's width is the next power of
    two, so that it changes rarely while sequences grow.  `token_rows` (one per
    entry, each entry bringing one token): the tokens lie on the device, entry
    b's in row token_rows[b] of a tensor given to the step; the indices go last
    in the array."""
    from ..cache import native
    B = len(batch)
    if not B:
        raise StepError("a step needs at least one sequence")
    slots = np.fromiter((s.slot for s in batch), dtype=np.int32, count=B)
    n_new = np.fromiter((len(s.tokens) for s in batch), dtype=np.int32, count=B)
    n_want = np.fromiter((len(s.want) for s in batch), dtype=np.int32, count=B)
    N, NW = int(n_new.sum()), int(n_want.sum())
    try:
        tokens = np.fromiter((t for s in batch for t in s.tokens), dtype=np.int64, count=N)
        want = np.fromiter((w for s in batch for w in s.want), dtype=np.int64, count=NW)
    except (TypeError, ValueError) as e:
        raise StepError(f"tokens and wanted indices must be integers ({e})") from None
    if N and token_rows is None and (tokens.min() < -2 ** 31 or tokens.max() >= 2 ** 31):
        raise StepError(f"token id {int(tokens.max())} is outside the vocabulary of {vocab_size}")
    tokens, want = tokens.astype(np.int32), np.clip(want, -1, 2 ** 31 - 1).astype(np.int32)
    rows = None
    if token_rows is not None:
        if len(token_rows) != B:
            raise StepError("tokens on the device: one row index per entry, and one token per entry")
        rows = np.ascontiguousarray(np.asarray(token_rows, dtype=np.int32))
    G = len(cache.groups)
    cap = 3 * N + (B + 1) + 5 * B + NW + B * sum(min(g.ring_pages, max(1, 2 * cache.n_pages)) for g in cache.groups)
    flat = np.empty(cap, dtype=np.int32)
    sizes = np.zeros(12 + G, dtype=np.int32)
    info = np.zeros(8 + G, dtype=np.int64)
    n_out = ctypes.c_long(0)
    native.check(native.lib().tl_pack_step(
        cache._h, B, slots.ctypes.data, n_new.ctypes.data, tokens.ctypes.data, n_want.ctypes.data,
        want.ctypes.data, int(vocab_size), rows.ctypes.data if rows is not None else None, flat.ctypes.data,
        cap, sizes.ctypes.data, info.ctypes.data, ctypes.byref(n_out)))
    pieces = int(info[6])
    szs = sizes[:pieces].tolist()
    off = np.concatenate([[0], np.cumsum(szs)])
    flat = flat[:n_out.value]
    len_before, len_after, cu = flat[off[5]:off[6]], flat[off[6]:off[7]], flat[off[3]:off[4]]
    return PackedStep(
        flat=flat, sizes=szs, n_rows=int(info[0]), n_seqs=B, n_want=int(info[1]),
        strides=tuple(int(w) for w in info[7:7 + G]), all_single=bool(info[2]), max_new=int(info[3]),
        max_len_after=int(info[4]),
        host={"n_new": n_new.astype(np.int64), "len_before": len_before.astype(np.int64),
              "len_after": len_after.astype(np.int64), "cu": cu.astype(np.int64), "slots": slots.tolist(),
              "aligned_cols": int(info[5])})


def context_from(packed: PackedStep, dev: torch.Tensor, cache: Cache, dtype: torch.dtype, device,
                 workspace: Workspace) -> Tuple[StepContext, Optional[torch.Tensor], int]:
    """Views of the uploaded array `dev` as the context that the parts see."""
    views, off = [], 0
    for n in packed.sizes:
        views.append(dev[off:off + n])
        off += n
    B = packed.n_seqs
    ctx = StepContext(
        n_rows=packed.n_rows, n_seqs=B, dtype=dtype, device=device,
        tokens=views[0], row_pos=views[1], row_seq=views[2], cu_seqlens=views[3], slots=views[4],
        len_before=views[5], len_after=views[6], tile_off=views[8],
        tables={gi: views[9 + gi].view(B, w) for gi, w in enumerate(packed.strides)},
        all_single=packed.all_single, max_new=packed.max_new, max_len_after=packed.max_len_after,
        workspace=workspace, cache=cache, host=dict(packed.host))
    return ctx, (views[7] if packed.n_want else None), packed.n_want


def build_context(cache: Cache, batch: Sequence[SeqInput], vocab_size: int, dtype: torch.dtype, device,
                  workspace: Workspace) -> Tuple[StepContext, Optional[torch.Tensor], int]:
    """`pack_step`, one upload, `context_from`."""
    packed = pack_step(cache, batch, vocab_size)
    dev = torch.from_numpy(packed.flat).to(device, non_blocking=False)
    return context_from(packed, dev, cache, dtype, device, workspace)


@dataclass
class _Graph:
    """A captured single-token step: its input array, workspace and logits."""
    meta: torch.Tensor
    staging: torch.Tensor
    workspace: Workspace
    graph: object = None
    logits: Optional[torch.Tensor] = None
    uploaded: Optional[torch.cuda.Event] = None      # the last copy out of `staging`


class Engine:
    """A model, its cache and workspace.  `max_tokens` is the most positions
    that live sequences hold at any time, each rounded up to whole pages."""

    def __init__(self, model: Model, max_tokens: int, max_slots: Optional[int] = None,
                 use_graphs: bool = True, freeze_gc: bool = False):
        """`freeze_gc`: take every object alive now (the model's among them) out of the
        garbage collector's sight (`gc.freeze()`), so that its passes, a millisecond each every
        few steps, do not stall decoding.  It acts on the whole process, the caller's objects
        included: for programs that serve one model until they end (the command line, the bench)."""
        self.model = model
        self.device = model.device
        self.cache: Cache = model.make_cache(max_tokens, max_slots)
        self.runs = model.bind_cache(self.cache)
        self.workspace = Workspace(self.device)
        self.vocab_size = model.spec.vocab_size
        self.use_graphs = use_graphs
        self.max_graphs = 32
        self._graphs: Dict[tuple, _Graph] = {}
        self._seen: Dict[tuple, int] = {}            # shapes of steps with several tokens a sequence: times seen
        if freeze_gc:
            gc.collect()
            gc.freeze()

    def close(self) -> None:
        """Give back the cache's storage, the captured graphs and the workspace now.  The engine
        cannot step afterwards; the model stays loaded."""
        self._graphs.clear()
        self._seen.clear()
        self.workspace.clear()
        self.runs = []
        self.cache.close()

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

    def step(self, batch: Sequence[SeqInput], device_tokens: Optional[torch.Tensor] = None,
             token_rows: Optional[Sequence[int]] = None) -> torch.Tensor:
        """Run one step; returns float32 logits [number of wanted rows, V] in
        the order of the entries and of their `want` lists.  The tensor is a
        view of the engine's workspace: it is overwritten by a later step.

        `device_tokens` (int32 on the GPU, e.g. what the sampler just drew) with
        `token_rows`: every entry brings one token, entry b's is
        device_tokens[token_rows[b]] (the entries' own `tokens` are ignored), so
        that a step can be launched before the host has seen the last one's
        tokens.  Ids outside the vocabulary are read as 0.

        Steps of few rows are launch-bound (the host needs some 15 us a kernel, a
        step of 32 layers 5 ms whatever its rows).  Where the model's parts allow
        (`Model.may_capture`: their own kernels only, up to 128 rows), a step in
        which every sequence brings one token is captured as a HIP graph the second
        time its shape (batch size, page-table widths) is seen, and from then on
        replayed; a step in which sequences bring several tokens (a short prompt, a
        chunk) likewise from the third time its shape is seen, the first time
        running in the engine's shared workspace, since most such shapes never come
        again."""
        if device_tokens is not None:
            if token_rows is None:
                token_rows = list(range(len(batch)))
            if device_tokens.dtype != torch.int32 or not device_tokens.is_cuda or not device_tokens.is_contiguous():
                raise StepError("device_tokens must be a contiguous int32 tensor on the GPU")
            if any(not (0 <= r < device_tokens.numel()) for r in token_rows):
                raise StepError(f"token_rows outside the {device_tokens.numel()} tokens on the device")
        elif token_rows is not None:
            raise StepError("token_rows without device_tokens")
        packed = pack_step(self.cache, batch, self.vocab_size, token_rows)
        growth = [(s.slot, len(s.tokens)) for s in batch]
        if (self.use_graphs and self.model.may_capture(packed.n_rows)
                and (packed.all_single or not self.model.prefers_eager(packed.host["n_new"], packed.host["len_before"],
                                                                        self.device))
                and (packed.all_single or self._seen_before(packed))):
            logits = self._graph_step(packed, device_tokens)
        else:
            dev = torch.from_numpy(packed.flat).to(self.device, non_blocking=False)
            self._take_tokens(packed, dev, device_tokens)
            ctx, want_rows, n_want = context_from(packed, dev, self.cache, self.model.dtype,
                                                  self.device, self.workspace)
            logits = self.model.forward(ctx, self.runs, want_rows, n_want)
        self.cache.commit(growth)
        return logits

    def _seen_before(self, packed: PackedStep) -> bool:
        """Count a shape of a step with several tokens a sequence; has it been seen before?"""
        key = packed.key
        n = self._seen.get(key, 0)
        if n == 0 and len(self._seen) >= 4096:
            self._seen.clear()
        self._seen[key] = n + 1
        return n > 0

    def _take_tokens(self, packed: PackedStep, dev: torch.Tensor, device_tokens: Optional[torch.Tensor]) -> None:
        """Fill the token section of the uploaded array from tokens on the device."""
        if device_tokens is None:
            return
        from ..kernels import ops
        B = packed.n_seqs
        ops.take_tokens(device_tokens, dev[dev.numel() - B:], self.vocab_size, dev[:B])

    def _graph_step(self, packed: PackedStep, device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        key = packed.key + (device_tokens is not None,)
        g = self._graphs.get(key)
        if g is None:
            # first sight: run it as it is, in the workspace the graph will own, so that
            # every buffer exists before the capture
            if len(self._graphs) >= self.max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
            g = _Graph(meta=torch.empty(packed.flat.size, dtype=torch.int32, device=self.device),
                       staging=torch.empty(packed.flat.size, dtype=torch.int32).pin_memory(),
                       workspace=Workspace(self.device))
            self._graphs[key] = g
        if g.uploaded is not None:
            g.uploaded.synchronize()                 # the staging area is free to be written again
        g.staging.numpy()[:] = packed.flat
        g.meta.copy_(g.staging, non_blocking=True)
        if g.uploaded is None:
            g.uploaded = torch.cuda.Event()
        g.uploaded.record()
        self._take_tokens(packed, g.meta, device_tokens)
        if g.graph is None and g.logits is not None:
            ctx, want_rows, n_want = context_from(packed, g.meta, self.cache, self.model.dtype,
                                                  self.device, g.workspace)
            ctx.host["fixed_launches"] = True        # replays come with other lengths
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                g.logits = self.model.forward(ctx, self.runs, want_rows, n_want)
            g.graph = graph
        if g.graph is not None:
            g.graph.replay()
            return g.logits
        ctx, want_rows, n_want = context_from(packed, g.meta, self.cache, self.model.dtype, self.device,
                                              g.workspace)
        ctx.host["fixed_launches"] = True            # the same launches as the capture that follows
        g.logits = self.model.forward(ctx, self.runs, want_rows, n_want)
        return g.logits
