"""Binding checkpoint tensors to a model's parts by name.

The model says which tensors it expects (name, shape, required or optional,
floating or integer); the loader checks the files against that list before a
single byte goes to the device and raises ONE error that lists every missing
tensor, every unexpected tensor and every wrong shape.  Tensors keep their
stored precision: bfloat16 stays bfloat16, a tensor stored in 32-bit stays
32-bit, half precision is widened to 32-bit (exactly); integer tables become
int32.  What the engine's dtype then needs is the parts' business.
"""
from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Dict, List, Tuple

import torch

from .safetensors_io import SafetensorsFile


@dataclass(frozen=True)
class ParamSpec:
    shape: Tuple[int, ...]
    required: bool = True
    integer: bool = False


class WeightError(RuntimeError):
    """Raised once per load, with all findings."""

    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}):")
            lines += [f"    - {n}" for n in self.missing]
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}):")
            lines += [f"    - {n}" for n in self.unexpected]
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}):")
            lines += [f"    - {n}: expected {list(want)}, found {list(got)}"
                      for n, want, got in self.wrong_shape]
        if self.wrong_dtype:
            lines.append(f"  wrong dtypes ({len(self.wrong_dtype)}):")
            lines += [f"    - {n}: {why}" for n, why in self.wrong_dtype]
        super().__init__("\n".join(lines))


_FLOAT_ST = {"F32", "F16", "BF16", "F64"}
_INT_ST = {"I64", "I32", "I16", "I8", "U8"}


def check_entries(expected: Dict[str, ParamSpec], found: Dict[str, Tuple[str, Tuple[int, ...]]],
                  ignorable: Callable[[str], bool] = lambda name: False) -> None:
    """Compare the expected tensors with the files' headers; raise WeightError
    with everything that is wrong.  `ignorable(name)` marks stored tensors that
    hold no weights (rotary tables that some exporters write)."""
    missing = [n for n, p in expected.items() if p.required and n not in found]
    unexpected = [n for n in found if n not in expected and not ignorable(n)]
    wrong_shape, wrong_dtype = [], []
    for n, (dt, shape) in found.items():
        if n not in expected:
            continue
        if tuple(shape) != tuple(expected[n].shape):
            wrong_shape.append((n, expected[n].shape, shape))
        if expected[n].integer and dt not in _INT_ST:
            wrong_dtype.append((n, f"expected an integer table, found {dt}"))
        if not expected[n].integer and dt not in _FLOAT_ST:
            wrong_dtype.append((n, f"expected floating point, found {dt}"))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(sorted(missing), sorted(unexpected), sorted(wrong_shape), sorted(wrong_dtype))


def stored_precision(t: torch.Tensor, integer: bool) -> torch.Tensor:
    """bfloat16 and float32 stay; float16 and float64 become float32; integer
    tables become int32."""
    if integer:
        return t.to(torch.int32)
    if t.dtype in (torch.bfloat16, torch.float32):
        return t
    return t.to(torch.float32)


class CheckpointFolder:
    """Every *.safetensors file of a folder, sorted by name
    (python/llaisys/models/qwen2.py:133), as one name -> tensor mapping."""

    def __init__(self, model_dir):
        self.dir = Path(model_dir)
        paths = sorted(self.dir.glob("*.safetensors"))
        if not paths:
            raise FileNotFoundError(f"no *.safetensors file in {self.dir}")
        self.files: List[SafetensorsFile] = [SafetensorsFile(p) for p in paths]
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        self._where: Dict[str, SafetensorsFile] = {}
        for f in self.files:
            for n, meta in f.entries.items():
                self.entries[n] = meta
                self._where[n] = f

    def tensor(self, name: str) -> torch.Tensor:
        return self._where[name].tensor(name)

    def close(self) -> None:
        for f in self.files:
            f.close()


def _is_rotary_table(name: str) -> bool:
    return name.endswith("rotary_emb.inv_freq")


def load_into(model, model_dir) -> None:
    """Check the folder against `model.expected_params()` and hand each part its
    tensors (`model.load_params(get)`, where get(name) returns the stored tensor
    on the CPU or None for an optional tensor that is absent)."""
    ckpt = CheckpointFolder(model_dir)
    try:
        expected = model.expected_params()
        check_entries(expected, ckpt.entries, _is_rotary_table)

        def get(name: str):
            if name not in ckpt.entries:
                return None
            return stored_precision(ckpt.tensor(name), expected[name].integer)

        model.load_params(get)
    finally:
        ckpt.close()
