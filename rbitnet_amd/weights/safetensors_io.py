"""Reading and writing the safetensors container, with nothing but the standard
library and torch.

File layout: 8 bytes little-endian header length n, n bytes of JSON
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`,
then the byte blob the offsets point into.

The reader is as defensive as the reference's GGUF parser
(crates/bitnet-core/src/gguf/parse.rs:88-196: magic and counts are checked
against sanity caps :103-115, every payload slice against the file's length
:65-80): header length within the file, offsets in range and ordered, byte
count equal to the product of the shape times the element size, no overlap.
An element type the engine cannot use is an error in the manner of
`UnsupportedGgmlType` (error.rs:25).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Optional, Tuple

import torch

from ..errors import WeightError

_DTYPES = {
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
_MAX_HEADER = 256 << 20      # sanity cap, as parse.rs:103-115 caps its counts


class SafetensorsFile:
    """One file, memory-mapped; tensors are views into the mapping."""

    def __init__(self, path: str):
        self.path = path
        try:
            size = os.path.getsize(path)
            self._fh = open(path, "rb")
        except OSError as e:
            raise WeightError(f"cannot open {path}: {e}") from None
        if size < 8:
            raise WeightError(f"{path}: too short to be a safetensors file ({size} bytes)")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen > _MAX_HEADER or 8 + hlen > size:
            raise WeightError(f"{path}: header length {hlen} exceeds the file ({size} bytes)")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightError(f"{path}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise WeightError(f"{path}: header is not a JSON object")
        self.metadata = header.pop("__metadata__", {}) or {}
        self.data_start = 8 + hlen
        self.data_len = size - self.data_start
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        spans: List[Tuple[int, int, str]] = []
        for name, info in header.items():
            try:
                dtype = info["dtype"]
                shape = tuple(int(s) for s in info["shape"])
                begin, end = (int(x) for x in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightError(f"{path}: malformed entry for tensor {name!r}") from None
            if dtype not in _DTYPES:
                raise WeightError(
                    f"{path}: unsupported element type {dtype} of tensor {name!r} "
                    f"(supported: {', '.join(sorted(_DTYPES))})")
            count = 1
            for s in shape:
                if s < 0:
                    raise WeightError(f"{path}: negative dimension in tensor {name!r}")
                count *= s
            if not 0 <= begin <= end <= self.data_len:
                raise WeightError(f"{path}: tensor {name!r} lies outside the file ({begin}..{end} of {self.data_len})")
            if end - begin != count * _DTYPES[dtype][1]:
                raise WeightError(
                    f"{path}: tensor {name!r} has {end - begin} bytes, its shape {list(shape)} "
                    f"of {dtype} needs {count * _DTYPES[dtype][1]}")
            self.entries[name] = (dtype, shape, begin, end)
            if end > begin:
                spans.append((begin, end, name))
        spans.sort()
        for (b0, e0, n0), (b1, e1, n1) in zip(spans, spans[1:]):
            if b1 < e0:
                raise WeightError(f"{path}: tensors {n0!r} and {n1!r} overlap")
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> List[str]:
        return list(self.entries)

    def info(self, name: str) -> Tuple[str, Tuple[int, ...]]:
        dtype, shape, _, _ = self.entries[name]
        return dtype, shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor in the stored element type (a copy is not made; the
        mapping stays alive as long as the tensor)."""
        dtype, shape, begin, end = self.entries[name]
        tdtype, _ = _DTYPES[dtype]
        if end == begin:
            return torch.empty(shape, dtype=tdtype)
        view = memoryview(self._mm)[self.data_start + begin:self.data_start + end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")          # torch warns that the buffer is read-only
            t = torch.frombuffer(view, dtype=tdtype)
        return t.reshape(shape)

    def close(self) -> None:
        # tensors handed out keep the mapping alive; only the descriptor is closed
        try:
            self._fh.close()
        except OSError:
            pass


class WeightFolder:
    """model.safetensors, or the shards model.safetensors.index.json lists."""

    def __init__(self, folder: str):
        self.folder = folder
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        self.files: List[SafetensorsFile] = []
        self.where: Dict[str, SafetensorsFile] = {}
        if os.path.isfile(folder):
            paths = [folder]
        elif os.path.isfile(single):
            paths = [single]
        elif os.path.isfile(index):
            with open(index) as f:
                try:
                    weight_map = json.load(f)["weight_map"]
                except (json.JSONDecodeError, KeyError, TypeError):
                    raise WeightError(f"{index}: not a shard index (no 'weight_map')") from None
            paths = []
            for shard in sorted(set(weight_map.values())):
                if os.path.basename(shard) != shard:
                    raise WeightError(f"{index}: shard name {shard!r} must be a plain file name")
                paths.append(os.path.join(folder, shard))
        else:
            raise WeightError(f"no model.safetensors (or model.safetensors.index.json) in {folder}")
        for p in paths:
            sf = SafetensorsFile(p)
            self.files.append(sf)
            for n in sf.names():
                if n in self.where:
                    raise WeightError(f"tensor {n!r} is stored twice ({self.where[n].path} and {p})")
                self.where[n] = sf

    def names(self) -> List[str]:
        return list(self.where)

    def info(self, name: str) -> Tuple[str, Tuple[int, ...]]:
        return self.where[name].info(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self.where[name].tensor(name)


def save_file(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata: Optional[Dict[str, str]] = None,
              layout: Optional[Dict[str, Tuple[torch.dtype, Tuple[int, ...]]]] = None) -> None:
    """Write tensors in the order given.  `tensors` may be a generator, so that a
    large model never sits in memory at once: then `layout` must give every
    tensor's element type and shape beforehand, for the header."""
    if layout is None:
        tensors = list(tensors)
        layout = {n: (t.dtype, tuple(t.shape)) for n, t in tensors}
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, (dtype, shape) in layout.items():
        if dtype not in _NAMES:
            raise WeightError(f"cannot store element type {dtype} of tensor {name!r}")
        count = 1
        for s in shape:
            count *= int(s)
        nbytes = count * _DTYPES[_NAMES[dtype]][1]
        header[name] = {"dtype": _NAMES[dtype], "shape": [int(s) for s in shape],
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        written = []
        for name, t in tensors:
            dtype, shape = layout[name]
            if t.dtype != dtype or tuple(t.shape) != tuple(shape):
                raise WeightError(f"tensor {name!r} does not match the announced layout")
            t = t.detach().to("cpu").contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
            written.append(name)
        if written != list(layout):
            raise WeightError("tensors were not written in the announced order")
    os.replace(tmp, path)
