"""Reading and writing the safetensors container.

The format is an 8-byte little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets"}}`` (``__metadata__`` skipped) and
the raw little-endian tensor bytes (reference: src/frontend/loader/safetensor.cpp:90-150
for the header and dtype table, :224-241 for the bounds checks, :268-304 for the
folder scan).  Files are memory-mapped; a tensor's bytes are only touched when
it is asked for.
"""
from __future__ import annotations

import glob
import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Mapping, Tuple

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


# name -> (bytes per element, numpy dtype used to view the bytes, torch dtype)
_DTYPES = {
    "F32": (4, np.float32, torch.float32),
    "F16": (2, np.float16, torch.float16),
    "BF16": (2, np.uint16, torch.bfloat16),
    "F64": (8, np.float64, torch.float64),
    "I64": (8, np.int64, torch.int64),
    "I32": (4, np.int32, torch.int32),
    "I16": (2, np.int16, torch.int16),
    "I8": (1, np.int8, torch.int8),
    "U8": (1, np.uint8, torch.uint8),
    "BOOL": (1, np.bool_, torch.bool),
}
_TORCH_TO_NAME = {v[2]: k for k, v in _DTYPES.items()}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int   # byte offsets inside the data section
    end: int
    path: str


class SafetensorsFile:
    """One memory-mapped ``.safetensors`` file."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file ({size} bytes)")
        self._f = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen <= 0 or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from e
        self.data_start = 8 + hlen
        self.data_size = size - self.data_start
        self.entries: Dict[str, TensorEntry] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            dt = info.get("dtype")
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dt!r}")
            shape = tuple(int(s) for s in info.get("shape", ()))
            off = info.get("data_offsets")
            if not (isinstance(off, list) and len(off) == 2):
                raise SafetensorsError(f"{path}: tensor '{name}' has no valid data_offsets")
            b, e = int(off[0]), int(off[1])
            nbytes = _DTYPES[dt][0] * int(np.prod(shape, dtype=np.int64)) if shape else _DTYPES[dt][0]
            if b < 0 or e < b or e - b != nbytes:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' spans bytes [{b},{e}) but dtype {dt} with shape "
                    f"{list(shape)} needs {nbytes}")
            if e > self.data_size:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' ends at byte {e}, past the data section ({self.data_size} bytes)")
            self.entries[name] = TensorEntry(name, dt, shape, b, e, path)
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self) -> List[str]:
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        """The tensor as a CPU torch tensor that owns a copy of its bytes."""
        e = self.entries[name]
        _, npdt, tdt = _DTYPES[e.dtype]
        count = int(np.prod(e.shape, dtype=np.int64)) if e.shape else 1
        arr = np.frombuffer(self._mm, dtype=npdt, count=count, offset=self.data_start + e.begin)
        t = torch.from_numpy(arr.copy())
        if e.dtype == "BF16":
            t = t.view(torch.bfloat16)
        return t.reshape(e.shape)

    def close(self) -> None:
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._f.close()


class SafetensorsFolder:
    """All ``*.safetensors`` of a folder, sorted by name; a tensor that several
    shards hold is taken from the last one (reference: safetensor.cpp:268-304)."""

    def __init__(self, folder: str):
        if not os.path.isdir(folder):
            raise SafetensorsError(f"model folder does not exist: {folder}")
        paths = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
        if not paths:
            raise SafetensorsError(f"no .safetensors file in {folder}")
        self.files = [SafetensorsFile(p) for p in paths]
        self.index: Dict[str, SafetensorsFile] = {}
        for f in self.files:
            for n in f.names():
                self.index[n] = f

    def names(self) -> List[str]:
        return list(self.index)

    def entry(self, name: str) -> TensorEntry:
        return self.index[name].entries[name]

    def tensor(self, name: str) -> torch.Tensor:
        return self.index[name].tensor(name)

    def close(self) -> None:
        for f in self.files:
            f.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor],
                      metadata: Mapping[str, str] | None = None) -> None:
    """Write tensors (moved to the CPU, made contiguous) as one safetensors file."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _TORCH_TO_NAME:
            raise SafetensorsError(f"cannot write tensor '{name}' of dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TORCH_TO_NAME[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().to("cpu").contiguous()
            if t.dtype == torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())
    os.replace(tmp, path)
