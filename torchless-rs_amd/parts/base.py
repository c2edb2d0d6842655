"""What a model is made of: parts, their registry, and the description of a
model as data.

A *part* is a mixer (attention, or anything else that mixes positions), a
feed-forward, a norm, a position encoding, or a block that arranges them.
Every part takes its sizes and constants as constructor parameters and knows
nothing about the model it sits in.  A model is a `ModelSpec`: for each layer
a `LayerSpec` naming the kind and parameters of its parts, and a schedule,
the list of layer indices in the order in which they run.  A layer may be
named twice (it then runs twice with the same weights and a cache of its own
for each run), and a run may read the cache that an earlier run wrote.

The reference hard-wires one arrangement (src/model/modules/layer.rs:28-56)
and one mixer; its per-architecture switches live in `ArchitectureConfig`
(src/model/architecture.rs:396-421, 487-502).  Here the switches are the
parts themselves.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

from ..weights.binding import WeightSpec

CATEGORIES = ("mixer", "ffn", "norm", "position", "block", "embedding", "head")
_PARTS: Dict[str, Dict[str, type]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, cls: type) -> None:
    if category not in _PARTS:
        raise KeyError(f"unknown part category {category!r}; there are {CATEGORIES}")
    _PARTS[category][kind] = cls


def unregister_part(category: str, kind: str) -> None:
    _PARTS[category].pop(kind, None)


def registered_parts(category: str) -> List[str]:
    return sorted(_PARTS[category])


@dataclass
class PartSpec:
    """Kind (a name in the registry) and constructor parameters of one part."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


def make_part(category: str, spec: PartSpec):
    kinds = _PARTS[category]
    if spec.kind not in kinds:
        raise KeyError(f"no {category} of kind {spec.kind!r}; registered: {sorted(kinds)}")
    return kinds[spec.kind](**spec.params)


@dataclass
class LayerSpec:
    prefix: str                       # the layer's tensors are named prefix + local name
    mixer: PartSpec
    ffn: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec
    block: PartSpec = field(default_factory=lambda: PartSpec("pre_norm"))


@dataclass
class Run:
    """One entry of the schedule: run `layer`; `kv_from`, if set, is the index
    of an earlier entry whose cache this run reads instead of owning one."""
    layer: int
    kv_from: Optional[int] = None


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    embedding_prefix: str
    layers: List[LayerSpec]
    schedule: List[Run]
    final_norm: PartSpec
    final_norm_prefix: str
    head: PartSpec
    head_prefix: str
    ignore_tensors: Tuple[str, ...] = ()

    def weight_specs(self) -> Dict[str, WeightSpec]:
        """Every tensor name the model binds, in a fixed order."""
        out: Dict[str, WeightSpec] = {}
        for k, v in make_part("embedding", self.embedding).weight_specs().items():
            out[self.embedding_prefix + k] = v
        for ls in self.layers:
            blk = make_part("block", PartSpec(ls.block.kind, dict(ls.block.params, layer=ls)))
            for k, v in blk.weight_specs().items():
                out[ls.prefix + k] = v
        for k, v in make_part("norm", self.final_norm).weight_specs().items():
            out[self.final_norm_prefix + k] = v
        for k, v in make_part("head", self.head).weight_specs().items():
            out.setdefault(self.head_prefix + k, v)
        return out


class Part:
    """Base of all parts.  `weight_specs` names the tensors it binds (local
    names); `load` receives them, already resident on the device in their
    stored width, and `compute_dtype` (float32 or bfloat16)."""

    # True if `forward` of a single-token step launches the same kernels with the same
    # arguments whatever the step's values are (everything that varies is read on the
    # device): such a step can be captured once as a HIP graph and replayed.
    graph_safe = False

    def may_capture(self, n_rows: int) -> bool:
        """May a single-token step of `n_rows` rows through this part go into a captured graph?
        A part whose kernels depend on the number of rows (a product that hands many rows to
        the BLAS library, whose launches stay out of graphs) answers for that number."""
        return self.graph_safe

    def prefers_eager(self, n_new, len_before, device) -> bool:
        """Would this part rather shape its launches by the lengths of this very step (sequences that
        bring `n_new` rows after `len_before` positions) than be replayed from a captured graph, whose
        launches are those of the step it was captured from?  A step that any part prefers eager is
        not captured."""
        return False

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], compute_dtype: torch.dtype) -> None:
        pass


@dataclass(frozen=True)
class RmsForm:
    """A norm of the form y = x * weight / sqrt(mean(x^2) + eps) over `size` channels."""
    weight: torch.Tensor          # float32 [size]
    size: int
    eps: float


class Norm(Part):
    def forward(self, ctx: "StepContext", x: torch.Tensor, out: torch.Tensor) -> None:
        """x: float32 [n, H] -> out [n, H] in the compute dtype."""
        raise NotImplementedError

    def rms_form(self) -> Optional[RmsForm]:
        """If the norm has the form of `RmsForm`, its terms: the products around it may then do
        its two halves (the sums of squares where the stream is completed, the factor per row
        on the results of the product that reads it).  None: the norm always runs by itself."""
        return None


class Position(Part):
    """A position encoding, as the attention mixer asks for it: how q and k are rotated."""

    def rotation(self, device):
        """An `ops.Rotation` (frequencies of the rotated pairs on `device`, how many of a head's
        channels are rotated, and whether pairs are halves apart or interleaved), or None if
        queries and keys are used as they are.  Keys enter the cache after the rotation, so
        any encoding that transforms a key by its own position alone fits this."""
        return None


class Mixer(Part):
    """A part that mixes information between positions of a sequence."""

    def kv_request(self):
        """A `KVRequest` if the mixer keeps keys and values per position."""
        return None

    def state_request(self):
        """A `StateRequest` if the mixer keeps a block of fixed size per sequence."""
        return None

    def forward(self, ctx: "StepContext", run: "RunBinding", y: torch.Tensor, x: torch.Tensor) -> None:
        """y: normed input [n, H] (compute dtype); ADD the result to x (float32 [n, H])."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx: "StepContext", y: torch.Tensor, x: torch.Tensor) -> None:
        """y: normed input [n, H]; ADD the result to x (float32 [n, H])."""
        raise NotImplementedError


@dataclass
class RunBinding:
    """What one run of the schedule owns or reads in the cache."""
    index: int
    kv_group: Any = None          # cache.KVGroup
    kv_group_index: int = -1
    kv_layer: int = 0             # layer index inside the group's storage
    kv_owner: bool = True         # False: reads another run's keys and values
    kv_source: int = -1           # the run that owns them (its own index for an owner)
    kv_read_later: bool = False   # a later run reads this run's keys and values
    state: Optional[torch.Tensor] = None      # [max_slots, *shape]


def take_row_factor(ctx: "StepContext", usable: bool):
    """For a part whose input came from a norm: the factor per row that its first product
    has to apply (None: the input is normed already).  A part that cannot apply it
    (`usable` false) gets the plain norm written into its input instead."""
    f = ctx.row_factor
    ctx.row_factor = None
    if f is not None and not usable:
        ctx.settle()
        f = None
    ctx.settle = None
    return f


def read_through_norm(ctx: "StepContext", norm: "Norm", x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """The stream `x` as `norm` gives it to the part behind it (a block calls this for every norm
    it runs; returns the buffer that holds the result, which is `y` or what a product left).
    Partial products that a part left pending are added first, by the norm itself if it can
    (`takes_pending`).  If the product that completed the stream did this norm's first half
    (`expect_norm` had announced it), the result is what that product left, and the factor per
    row goes to the part that reads it (`ctx.row_factor`; `ctx.settle` runs the plain norm into
    the same buffer for a part that cannot apply it)."""
    pre, ctx.prenormed = ctx.prenormed, None
    if pre is not None and pre[0] is norm:
        ctx.row_factor = pre[2]
        ctx.settle = lambda: norm.forward(ctx, x, pre[1])
        return pre[1]
    if not getattr(norm, "takes_pending", False):
        flush_pending(ctx, x)
    norm.forward(ctx, x, y)
    return y


def expect_norm(ctx: "StepContext", writer: Part, norm: Optional["Norm"], reader: Optional[Part] = None) -> None:
    """Before `writer` runs: announce that `norm` reads the stream next and `reader` reads the
    norm.  If all three can (`writer.closes_stream`, `norm.rms_form()`, `reader.takes_row_factor`)
    the product that completes the stream may do the norm's first half (steps of at most 16
    rows); if not, nothing is announced and the norm runs by itself.  `reader` None: the norm
    is another block's `splittable_entry`, which has asked its reader already."""
    ok = (norm is not None and getattr(writer, "closes_stream", False) and norm.rms_form() is not None
          and (reader is None or getattr(reader, "takes_row_factor", False)))
    ctx.norm_ahead = norm if ok else None


def part_done(ctx: "StepContext", part: Part) -> None:
    """After a part has run: what was announced to it is void, and a factor per row that it was
    handed must have been taken."""
    ctx.norm_ahead = None
    if ctx.row_factor is not None:
        raise RuntimeError(f"{type(part).__name__} declares takes_row_factor and left the factor untaken")


def splittable_entry(norm: "Norm", reader: Part) -> Optional["Norm"]:
    """`norm` if it is the first reader of the stream in a block and can be cut in two for
    `reader` (the block before may then do its first half); else None."""
    return norm if norm.rms_form() is not None and getattr(reader, "takes_row_factor", False) else None


def flush_pending(ctx: "StepContext", x: torch.Tensor) -> None:
    """Add partial products that a part left in `ctx.pending` to the stream."""
    if ctx.pending is not None:
        from ..kernels import ops
        ops.add_partials(x, ctx.pending)
        ctx.pending = None


class Workspace:
    """Scratch tensors by name, kept between steps so that a step allocates
    nothing once sizes have been seen (and a captured graph keeps its
    addresses)."""

    def __init__(self, device):
        self.device = device
        self._bufs: Dict[str, torch.Tensor] = {}
        self._views: Dict[tuple, torch.Tensor] = {}      # (name, dtype, shape) -> the view handed out last time

    def get(self, name: str, shape: Tuple[int, ...], dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
        """`zero`: the buffer is zero when it is first made (not on later calls:
        for counters that their kernels leave at zero)."""
        shape = tuple(int(s) for s in shape)
        at = (name, dtype, shape)
        view = self._views.get(at)
        if view is not None:                # every layer of a step asks for the same few
            return view
        n = 1
        for s in shape:
            n *= s
        key = f"{name}:{dtype}"
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            make = torch.zeros if zero else torch.empty
            buf = make(max(n, 1), dtype=dtype, device=self.device)
            self._bufs[key] = buf
            for k in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[k]          # views of the buffer that this one replaces
        view = buf[:n].view(shape)
        if len(self._views) > 4096:
            self._views.clear()
        self._views[at] = view
        return view

    def clear(self) -> None:
        self._bufs.clear()
        self._views.clear()


@dataclass
class StepContext:
    """One step's batch as the parts see it.  Rows are the tokens of all
    sequences, packed sequence after sequence."""
    n_rows: int
    n_seqs: int
    dtype: torch.dtype                    # compute dtype of activations and cache
    device: Any
    tokens: torch.Tensor                  # int32 [n]
    row_pos: torch.Tensor                 # int32 [n]  position of the row in its sequence
    row_seq: torch.Tensor                 # int32 [n]  index of the row's sequence in this batch
    cu_seqlens: torch.Tensor              # int32 [B+1]
    slots: torch.Tensor                   # int32 [B]
    len_before: torch.Tensor              # int32 [B]
    len_after: torch.Tensor               # int32 [B]
    tile_off: torch.Tensor                # int32 [B]  column of each sequence in buffers laid out by
                                          #   `ops.aligned_columns` (host["aligned_cols"] in all)
    tables: Dict[int, torch.Tensor]       # group index -> int32 [B, stride] page ids
    all_single: bool                      # every sequence brings exactly one token
    max_new: int
    max_len_after: int
    workspace: Workspace
    cache: Any
    # partial products [S, n, H] (float32) that still have to be added to the residual stream:
    # a product may leave them here instead of adding them itself; whoever reads the stream
    # next (a norm that can, else `flush`) adds them up
    pending: Optional[torch.Tensor] = None
    # An RMSNorm may be cut in two around the products next to it (steps of at most 16 rows):
    # `norm_ahead` is the norm that reads the stream next, set by whoever knows it while a
    # part runs whose last write to the stream is `Linear.add_into` (`closes_stream`), which
    # may then do the norm's first half; `prenormed` is what such a
    # product left: (norm, x * weight in the compute dtype, `ops.RowFactor`); `row_factor`
    # is handed by the norm to the part that reads its output, which must take it
    # (`take_row_factor`) and pass it to its first product, or ask `settle` for the plain norm
    norm_ahead: Any = None
    prenormed: Any = None
    row_factor: Any = None
    settle: Any = None
    host: Dict[str, Any] = field(default_factory=dict)     # the same data on the host
