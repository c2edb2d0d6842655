"""Grouped-query attention over the cache, with an optional sliding window.

q = Wq y, k = Wk y, v = Wv y (no bias); q and k rotated by the position
encoding before k enters the cache; query head h reads KV head h // (nq/nkv);
score = (k.q) / sqrt(d); softmax over the visible keys; output projection
(src/model/modules/attention.rs:42-135 of the reference).  Key j is visible
to the query at p iff j <= p and, with a window W, j > p - W
(src/model/models/gpt_oss.rs:168-175; the reference's Mistral path reads the
window from the file and never applies it).

The three projections are bound under their own names (`names`: the leaf names
are parameters, and a checkpoint that stores q|k|v as one tensor binds that one)
and laid side by side at load so that one product serves them.  How q and k
are rotated is the position part's answer (`Position.rotation`: frequencies, how
many channels of a head, which pairing; or no rotation at all); the mixer hands
it to the kernels and knows no formula of it.  Rows of a step that bring more
than one token attend to the cache for older positions and to the step's own
keys for the new ones, and the keys are committed afterwards; single-token
steps commit first and read everything from the cache.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..cache.cache import KVRequest
from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Mixer, PartSpec, make_part, register_part, take_row_factor
from .linear import Linear


class AttentionMixer(Mixer):
    graph_safe = True
    closes_stream = True          # its last write to the stream is `Linear.add_into`
    takes_row_factor = True       # its q|k|v product can do the division of the norm before it

    # leaf names of the tensors under `prefix`; "qkv": one tensor [q | k | v] by rows instead of the three
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "qkv": None}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: PartSpec, window: Optional[int] = None, own_kv: bool = True,
                 prefix: str = "self_attn.", names: Optional[Dict[str, Optional[str]]] = None,
                 scale: Optional[float] = None):
        """`scale`: what a score k.q is multiplied by before the softmax; None: 1 / sqrt(head_dim)."""
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} KV heads")
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"attention: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        if self.names["qkv"] and not own_kv:
            raise ValueError("attention: a mixer that reads another's keys and values binds q alone, not q|k|v")
        self.H, self.nq, self.nkv, self.d = int(hidden_size), int(n_heads), int(n_kv_heads), int(head_dim)
        self.window = int(window) if window else None
        self.own_kv = bool(own_kv)
        self.prefix = prefix
        self.position = make_part("position", position)
        self.scale = 1.0 / math.sqrt(self.d) if scale is None else float(scale)
        self.qkv = None
        self.o = None

    def kv_request(self):
        return KVRequest(self.nkv, self.d, self.window) if self.own_kv else None

    def may_capture(self, n_rows: int) -> bool:
        return self.qkv is not None and self.qkv.own_kernels(n_rows) and self.o.own_kernels(n_rows)

    def prefers_eager(self, n_new, len_before, device) -> bool:
        # few rows over a long context: the host cuts the keys into runs for workgroups of their own
        return (self.qkv is not None and ops.prefill_serves(self.qkv.weight.dtype, self.d)
                and ops.prefill_layout(n_new, len_before, self.window, self.nq, ops.compute_units(device)) is not None)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        if nm["qkv"]:
            out = {p + nm["qkv"]: WeightSpec(((self.nq + 2 * self.nkv) * self.d, self.H))}
        else:
            out = {p + nm["q"]: WeightSpec((self.nq * self.d, self.H))}
            if self.own_kv:
                out[p + nm["k"]] = WeightSpec((self.nkv * self.d, self.H))
                out[p + nm["v"]] = WeightSpec((self.nkv * self.d, self.H))
        out[p + nm["o"]] = WeightSpec((self.H, self.nq * self.d))
        return out

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names
        if nm["qkv"]:
            fused = tensors[p + nm["qkv"]]
        else:
            ws = [tensors[p + nm["q"]]]
            if self.own_kv:
                ws += [tensors[p + nm["k"]], tensors[p + nm["v"]]]
            if len({w.dtype for w in ws}) > 1:
                ws = [w.to(torch.float32) for w in ws]
            fused = torch.cat(ws, dim=0)
        # single-token steps stream q|k|v and o from tiled copies; the fused q|k|v kernel has its own
        # order of rows, which follows the pairs of the rotation
        rows = None
        if self.own_kv and self.d % 16 == 0 and fused.is_cuda and fused.dtype == torch.bfloat16:
            rows = ops.qkv_tile_rows(self.nq, self.nkv, self.d, fused.device,
                                     self.position.rotation(fused.device) or ops.NO_ROTATION)
        self.qkv = Linear(fused, tiled=True, tile_rows=rows)
        self.o = Linear(tensors[p + nm["o"]], tiled=True)

    def forward(self, ctx, run, y: torch.Tensor, x: torch.Tensor) -> None:
        n, nq, nkv, d = y.shape[0], self.nq, self.nkv, self.d
        ws = ctx.workspace
        group = run.kv_group
        pages = group.storage[run.kv_layer]
        table = ctx.tables[run.kv_group_index]
        rotation = self.position.rotation(y.device) or ops.NO_ROTATION
        q = ws.get("attn_q", (n, nq, d), ctx.dtype)
        out = ws.get("attn_out", (n, nq, d), ctx.dtype)
        fused = (self.own_kv and ctx.all_single and not run.kv_read_later
                 and ops.qkv_rope_commit_ok(y, self.qkv.weight, d, pages))
        factor = take_row_factor(ctx, usable=fused)
        if self.own_kv and ctx.all_single and not run.kv_read_later:
            # one token a sequence: k and v go straight into the pages, then everything is read there
            if fused:
                ops.qkv_rope_commit(y, self.qkv.weight, ctx.row_pos, rotation, table, group.ring_pages,
                                    nq, nkv, d, q, pages, factor=factor,     # product, rotation and commit in one
                                    tiles=self.qkv.own_tiles)
            else:
                qkv = self.qkv.partial(y, ctx, "attn_qkv_parts")     # partial sums, added up by the rotation
                if qkv is None:
                    qkv = ws.get("attn_qkv", (n, (nq + 2 * nkv) * d), torch.float32)
                    self.qkv(y, qkv)
                ops.rope_commit(qkv, ctx.row_pos, rotation, table, group.ring_pages, nq, nkv, d, q, pages)
            ops.attention(q, None, None, pages, table, group.ring_pages, ctx, ctx.len_after,
                          self.window, self.scale, out)
            self.o.add_into(out.view(n, nq * d), x, ctx, "attn_o_parts")
            return
        if self.own_kv:
            tag = f"_{run.index}" if run.kv_read_later else ""
            parts = self.qkv.partial(y, ctx, "attn_qkv_parts")
            if parts is not None:               # K cut into partial sums: the first slice takes the others
                qkv = parts[0]
                ops.add_partials(qkv, parts[1:])
            else:
                qkv = ws.get("attn_qkv", (n, (nq + 2 * nkv) * d), torch.float32)
                self.qkv(y, qkv)
            k = ws.get("attn_k" + tag, (n, nkv, d), ctx.dtype)
            if ops.uses_transposed_values(ctx.dtype, d, ctx.all_single):
                # the matrix cores read values along the keys: only the transposed copy is made, by tiles
                v = None
                vt = ws.get("attn_vt" + tag, (nkv, d, ctx.host["aligned_cols"]), ctx.dtype)
                ops.rope_v_tiles(qkv, ctx.row_pos, rotation, nq, nkv, d, q, k, vt, ctx.cu_seqlens, ctx.tile_off,
                                 ctx.len_before, ctx.len_after)       # rotation and transposition in one launch
            else:
                vt = None
                v = ws.get("attn_v" + tag, (n, nkv, d), ctx.dtype)
                ops.rope_split(qkv, ctx.row_pos, rotation, nq, nkv, d, q, k, v)
            if run.kv_read_later:
                ctx.host[f"kv_new_{run.index}"] = (k, v, vt)
        else:
            qf = ws.get("attn_qkv", (n, nq * d), torch.float32)
            self.qkv(y, qf)
            ops.rope_split(qf, ctx.row_pos, rotation, nq, 0, d, q, None, None)
            k, v, vt = ctx.host[f"kv_new_{run.kv_source}"]
        if ctx.all_single and not self.own_kv:
            ops.attention(q, None, None, pages, table, group.ring_pages, ctx, ctx.len_after,
                          self.window, self.scale, out)
        elif ctx.all_single:
            ops.kv_commit(k, v, ctx.row_seq, ctx.row_pos, ctx.len_after, table, group.ring_pages, pages)
            ops.attention(q, None, None, pages, table, group.ring_pages, ctx, ctx.len_after,
                          self.window, self.scale, out)
        else:
            ops.attention(q, k, v, pages, table, group.ring_pages, ctx, ctx.len_before,
                          self.window, self.scale, out, vt_new=vt)
            if self.own_kv:
                def commit():
                    if vt is not None:
                        ops.kv_commit_tiles(k, vt, ctx.row_seq, ctx.row_pos, ctx.tile_off, ctx.len_before,
                                            ctx.len_after, table, group.ring_pages, pages)
                    else:
                        ops.kv_commit(k, v, ctx.row_seq, ctx.row_pos, ctx.len_after, table,
                                      group.ring_pages, pages)
                if run.kv_read_later:       # a later run still reads the old rows of the ring
                    ctx.host.setdefault("deferred", []).append(commit)
                else:
                    commit()
        self.o.add_into(out.view(n, nq * d), x, ctx, "attn_o_parts")


register_part("mixer", "attention", AttentionMixer)
