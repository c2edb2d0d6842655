"""Reading and writing safetensors files, by tensor name.

Format (as the reference reads it, src/loader/formats/safetensors.rs:6-25,
198-280, 336-356): a little-endian u64 header length, a JSON object
`{name: {dtype, shape, data_offsets: [begin, end]}, "__metadata__": {...}}`,
then the data; offsets count from the end of the header.  A folder may hold
one `model.safetensors` or shards named by `model.safetensors.index.json`.

Tensors come back as CPU torch tensors that alias a read-only memory map, in
the dtype the file stores; nothing is converted here.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Optional, Tuple

import torch


class SafetensorsError(ValueError):
    """A file that is not a well-formed safetensors file."""


_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One `.safetensors` file, memory-mapped."""

    def __init__(self, path: str):
        self.path = path
        try:
            size = os.path.getsize(path)
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"{path}: cannot open: {e}") from None
        if size < 8:
            raise SafetensorsError(f"{path}: shorter than the 8-byte header length")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if 8 + hlen > size:
            raise SafetensorsError(f"{path}: header of {hlen} bytes runs past the end of the file")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header must be a JSON object")
        self.metadata = header.pop("__metadata__", None) or {}
        self._base = 8 + hlen
        self._data_len = size - self._base
        self._info: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, e in header.items():
            try:
                dt, dims, (b, en) = e["dtype"], list(e["shape"]), e["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed entry for tensor {name!r}") from None
            if any(type(v) is not int for v in dims + [b, en]):
                raise SafetensorsError(f"{path}: tensor {name!r}: shape and data_offsets must be integers")
            if any(v < 0 for v in dims):
                raise SafetensorsError(f"{path}: tensor {name!r} has a negative dimension in {dims}")
            shape = tuple(dims)
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unknown dtype {dt!r}")
            n = 1
            for s in shape:
                n *= s
            if not (0 <= b <= en <= self._data_len):
                raise SafetensorsError(
                    f"{path}: tensor {name!r} data_offsets [{b}, {en}] lie outside the file")
            if en - b != n * _DTYPES[dt][1]:
                raise SafetensorsError(
                    f"{path}: tensor {name!r} holds {en - b} bytes, its shape {list(shape)} and "
                    f"dtype {dt} need {n * _DTYPES[dt][1]}")
            self._info[name] = (dt, shape, int(b), int(en))
        end = 0
        for name, (_, _, b, en) in sorted(self._info.items(), key=lambda kv: kv[1][2:]):
            if b < end and en > b:
                raise SafetensorsError(f"{path}: the data of tensor {name!r} overlaps another tensor's")
            end = max(end, en)
        self._mm: Optional[mmap.mmap] = None

    def names(self) -> List[str]:
        return list(self._info)

    def __contains__(self, name: str) -> bool:
        return name in self._info

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._info[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._info[name][0]][0]

    def tensor(self, name: str) -> torch.Tensor:
        if name not in self._info:
            raise KeyError(f"{self.path}: tensor {name!r} not found")
        dt, shape, b, e = self._info[name]
        if e == b:
            return torch.empty(shape, dtype=_DTYPES[dt][0])
        if self._mm is None:
            self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")          # the map is read-only; nobody writes
            t = torch.frombuffer(self._mm, dtype=_DTYPES[dt][0], count=(e - b) // _DTYPES[dt][1],
                                 offset=self._base + b)
        return t.view(shape)


class ModelFiles:
    """All tensors of a model folder: one file, or the shards of an index."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.isfile(single):
            f = SafetensorsFile(single)
            self._files[single] = f
            for n in f.names():
                self._where[n] = single
        elif os.path.isfile(index):
            with open(index) as fh:
                try:
                    wm = json.load(fh)["weight_map"]
                except (json.JSONDecodeError, KeyError, TypeError):
                    raise SafetensorsError(f"{index}: no 'weight_map'") from None
            if not isinstance(wm, dict) or not all(isinstance(v, str) for v in wm.values()):
                raise SafetensorsError(f"{index}: 'weight_map' must map tensor names to file names")
            for shard in sorted(set(wm.values())):
                # a shard is a file of this folder: no path, no way out of it
                if os.path.basename(shard) != shard or shard in ("", ".", ".."):
                    raise SafetensorsError(f"{index}: shard name {shard!r} is not a plain file name")
                p = os.path.join(model_dir, shard)
                if os.path.dirname(os.path.realpath(p)) != os.path.realpath(model_dir):
                    raise SafetensorsError(f"{index}: shard {shard!r} lies outside {model_dir}")
                f = SafetensorsFile(p)
                self._files[p] = f
                for n in f.names():
                    self._where[n] = p
            lost = [n for n in wm if n not in self._where]
            if lost:
                raise SafetensorsError(f"{index}: names tensors that no shard holds: {lost[:8]}")
        else:
            raise SafetensorsError(
                f"{model_dir}: neither model.safetensors nor model.safetensors.index.json")

    def names(self) -> List[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._files[self._where[name]].shape(name)

    def dtype(self, name: str) -> torch.dtype:
        return self._files[self._where[name]].dtype(name)

    def tensor(self, name: str) -> torch.Tensor:
        if name not in self._where:
            raise KeyError(f"tensor {name!r} not found in {self.model_dir}")
        return self._files[self._where[name]].tensor(name)


class TensorDict:
    """The same interface over tensors that are already in memory."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self._t = tensors

    def names(self) -> List[str]:
        return list(self._t)

    def __contains__(self, name: str) -> bool:
        return name in self._t

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._t[name].shape)

    def dtype(self, name: str) -> torch.dtype:
        return self._t[name].dtype

    def tensor(self, name: str) -> torch.Tensor:
        return self._t[name]


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor],
                      metadata: Optional[Dict[str, str]] = None) -> None:
    """Write `tensors` (in the order given) as one safetensors file."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    items: List[Tuple[str, torch.Tensor]] = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [off, off + n]}
        off += n
        items.append((name, t))
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for _, t in items:
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                        t.reshape(1).view(torch.uint8).numpy().tobytes())
