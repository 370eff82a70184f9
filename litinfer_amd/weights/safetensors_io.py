"""Reading and writing the safetensors file format.

Layout (as the reference reads it by hand, python/llaisys/models/qwen2.py:112-129):
u64 little-endian header length, a JSON header {name: {dtype, shape,
data_offsets: [begin, end]}} (the entry `__metadata__` is skipped), then the
data section.  The file is memory-mapped; a tensor is a view until it is
copied to the device.  Offsets are checked against the file and the shape,
which the reference does not do.
"""
from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path
from typing import Dict, Iterable, Tuple

import numpy as np
import torch

# safetensors dtype -> (numpy dtype that carries the bits, torch dtype of the view)
_DTYPES = {
    "F32": (np.float32, torch.float32),
    "F16": (np.float16, torch.float16),
    "BF16": (np.int16, torch.bfloat16),
    "F64": (np.float64, torch.float64),
    "I64": (np.int64, torch.int64),
    "I32": (np.int32, torch.int32),
    "I16": (np.int16, torch.int16),
    "I8": (np.int8, torch.int8),
    "U8": (np.uint8, torch.uint8),
    "BOOL": (np.bool_, torch.bool),
}
_TORCH_TO_ST = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
                torch.float64: "F64", torch.int64: "I64", torch.int32: "I32",
                torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8", torch.bool: "BOOL"}


class SafetensorsFile:
    """A memory-mapped safetensors file: `entries` maps a tensor name to
    (dtype string, shape); `tensor(name)` gives a CPU tensor that views the map."""

    def __init__(self, path):
        self.path = Path(path)
        self._f = open(self.path, "rb")
        size = self.path.stat().st_size
        if size < 8:
            raise ValueError(f"{self.path}: too short for a safetensors file")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._mm[:8])
        if 8 + hlen > size:
            raise ValueError(f"{self.path}: header length {hlen} exceeds the file size {size}")
        header = json.loads(self._mm[8:8 + hlen].decode("utf-8"))
        self._base = 8 + hlen
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        self._offsets: Dict[str, Tuple[int, int]] = {}
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            dt, shape = meta["dtype"], tuple(int(s) for s in meta["shape"])
            if dt not in _DTYPES:
                raise ValueError(f"{self.path}: tensor '{name}' has unsupported safetensors dtype {dt}")
            b, e = (int(v) for v in meta["data_offsets"])
            numel = int(np.prod(shape, dtype=np.int64)) if shape else 1
            want = numel * np.dtype(_DTYPES[dt][0]).itemsize
            if e - b != want or b < 0 or self._base + e > size:
                raise ValueError(f"{self.path}: tensor '{name}' has data_offsets [{b}, {e}] but its "
                                 f"shape {list(shape)} and dtype {dt} need {want} bytes inside a "
                                 f"data section of {size - self._base}")
            self.entries[name] = (dt, shape)
            self._offsets[name] = (b, e)

    def tensor(self, name: str) -> torch.Tensor:
        dt, shape = self.entries[name]
        np_dt, torch_dt = _DTYPES[dt]
        b, e = self._offsets[name]
        count = (e - b) // np.dtype(np_dt).itemsize
        arr = np.frombuffer(self._mm, dtype=np_dt, count=count, offset=self._base + b)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")         # the map is read-only; the view is never written
            t = torch.from_numpy(arr)
        if torch_dt is torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def close(self) -> None:
        try:
            self._mm.close()
        except BufferError:
            pass                                     # views are still alive; the map goes with them
        self._f.close()


def write_safetensors(path, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write (name, tensor) pairs, in the given order.  Tensors are taken one at
    a time so that a large model never sits in memory twice."""
    tensors = list(tensors)
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    for name, t in tensors:
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _TORCH_TO_ST[t.dtype], "shape": list(t.shape),
                        "data_offsets": [off, off + n]}
        off += n
    hjson = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hjson += b" " * ((8 - len(hjson) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hjson)))
        f.write(hjson)
        for _, t in tensors:
            t = t.detach().cpu().contiguous()
            if t.dtype is torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())
