"""Reading and writing the safetensors container.

Format rules as kappai's parser states them (src/safetensors.c:9-66, 75-144): eight bytes
of little-endian header length, a JSON header ``{name: {dtype, shape, data_offsets}}``
in which ``__metadata__`` is skipped, then the tensors' bytes; ``data_offsets`` are
checked against the file size and against dtype x shape.
"""
from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from pathlib import Path
from typing import Dict, Iterable, Tuple

import numpy as np
import torch

DTYPE_BYTES = {"BF16": 2, "F16": 2, "F32": 4, "I32": 4, "I64": 8}
_TORCH_OF = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32,
             "I32": torch.int32, "I64": torch.int64}
_NAME_OF = {v: k for k, v in _TORCH_OF.items()}


class SafetensorsError(ValueError):
    pass


@dataclass
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int      # byte offsets into the file
    end: int


class SafetensorsFile:
    """A memory-mapped safetensors file: the header is parsed at once, tensors are read
    on demand so that a large checkpoint is never held in host memory twice."""

    def __init__(self, path):
        self.path = Path(path)
        if not self.path.is_file():
            raise SafetensorsError(f"{self.path}: no such file")
        size = self.path.stat().st_size
        with open(self.path, "rb") as f:
            head = f.read(8)
            if len(head) < 8:
                raise SafetensorsError(f"{self.path}: shorter than a safetensors header")
            (hlen,) = struct.unpack("<Q", head)
            if hlen <= 0 or 8 + hlen > size:
                raise SafetensorsError(f"{self.path}: header length {hlen} exceeds the file")
            try:
                header = json.loads(f.read(hlen))
            except (json.JSONDecodeError, UnicodeDecodeError) as exc:
                raise SafetensorsError(f"{self.path}: header is not JSON ({exc})") from exc
        if not isinstance(header, dict):
            raise SafetensorsError(f"{self.path}: header must be an object")
        base = 8 + hlen
        self.entries: Dict[str, TensorEntry] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                dtype = info["dtype"]
                shape = tuple(int(s) for s in info["shape"])
                lo, hi = (int(v) for v in info["data_offsets"])
            except (KeyError, TypeError, ValueError) as exc:
                raise SafetensorsError(f"{self.path}: malformed entry for '{name}'") from exc
            if dtype not in DTYPE_BYTES:
                raise SafetensorsError(f"{self.path}: tensor '{name}' has unsupported dtype {dtype}")
            count = 1
            for s in shape:
                count *= s
            if hi - lo != count * DTYPE_BYTES[dtype] or lo < 0 or base + hi > size:
                raise SafetensorsError(
                    f"{self.path}: tensor '{name}' ({dtype} {list(shape)}) does not fit its "
                    f"data_offsets [{lo}, {hi}) in a file of {size} bytes")
            self.entries[name] = TensorEntry(name, dtype, shape, base + lo, base + hi)
        last = None
        for e in sorted(self.entries.values(), key=lambda e: (e.begin, e.end)):
            if last is not None and e.begin < last.end:
                raise SafetensorsError(f"{self.path}: tensors '{last.name}' and '{e.name}' "
                                       "overlap in the file")
            if e.end > e.begin:
                last = e
        self._file = open(self.path, "rb")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def read(self, name: str) -> torch.Tensor:
        """The tensor as a CPU torch tensor of its stored dtype (a copy)."""
        e = self.entries[name]
        count = (e.end - e.begin) // DTYPE_BYTES[e.dtype]
        if count == 0:
            return torch.empty(e.shape, dtype=_TORCH_OF[e.dtype])
        if e.dtype == "BF16":
            raw = np.frombuffer(self._map, dtype="<i2", count=count, offset=e.begin).copy()
            t = torch.from_numpy(raw).view(torch.bfloat16)
        else:
            np_dt = {"F16": "<f2", "F32": "<f4", "I32": "<i4", "I64": "<i8"}[e.dtype]
            t = torch.from_numpy(np.frombuffer(self._map, dtype=np_dt, count=count,
                                               offset=e.begin).copy())
        return t.reshape(e.shape)

    def close(self):
        if self._map is not None:
            self._map.close()
            self._map = None
        self._file.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def write_safetensors(path, tensors: Dict[str, torch.Tensor], metadata=None) -> None:
    """Write CPU tensors in the order given; data is aligned as the header ends (padded
    with spaces to a multiple of 8 bytes)."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().contiguous().cpu()
        if t.dtype not in _NAME_OF:
            raise SafetensorsError(f"cannot store '{name}' of dtype {t.dtype}")
        if t.dtype == torch.bfloat16:
            raw = t.view(torch.int16).numpy().tobytes()
        else:
            raw = t.numpy().tobytes()
        header[name] = {"dtype": _NAME_OF[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    hjson = json.dumps(header, separators=(",", ":")).encode()
    hjson += b" " * ((8 - len(hjson) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hjson)))
        f.write(hjson)
        for raw in blobs:
            f.write(raw)
