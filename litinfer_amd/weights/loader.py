"""Binding checkpoint tensors to a model's parts by name.

The model says which tensors it expects (name, shape, required or optional,
floating or integer); the loader checks the files against that list before a
single byte goes to the device and raises ONE error that lists every missing
tensor and every wrong shape (and, when asked to be strict, every stored tensor
that the model does not know).  Stored names may be aliases that the
architecture declares; a stored tensor that the model does not use is counted
and reported in one line, as the reference lets unknown names fall through
(python/llaisys/models/qwen2.py:139-194).  The loader hands
tensors on in their stored precision: bfloat16 stays bfloat16, a tensor stored
in 32-bit stays 32-bit, half precision is widened to 32-bit (exactly); integer
tables become int32.  The model's runtime then binds every MATRIX in the
engine's one dtype (`parts.Runtime.matrix`: the reference converts every tensor
to the model's dtype, python/llaisys/models/qwen2.py:88-110, 253-264) and
holds norm weights and biases in 32-bit; when matrices had to be rounded for
that, one line says so.
"""
from __future__ import annotations

import sys
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Dict, List, Mapping, Optional, Tuple

import torch

from .safetensors_io import SafetensorsFile


INIT_KINDS = ("normal", "one_plus_normal", "zeros", "ones")


@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part expects.  `init` says how random weights draw it: "normal" is
    N(0, 0.02), "one_plus_normal" 1 + N(0, 0.02) (the weights of a norm), "zeros", "ones"."""
    shape: Tuple[int, ...]
    required: bool = True
    integer: bool = False
    init: str = "normal"

    def __post_init__(self):
        if self.init not in INIT_KINDS:
            raise ValueError(f"ParamSpec: init must be one of {INIT_KINDS}, found {self.init!r}")


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
                  ignorable: Callable[[str], bool] = lambda name: False, strict: bool = True) -> List[str]:
    """Compare the expected tensors with the files' headers; raise WeightError
    with everything that is wrong.  `ignorable(name)` marks stored tensors that
    hold no weights (rotary tables that some exporters write).  A stored tensor
    that is not expected is an error when `strict`; otherwise the names of such
    tensors are returned."""
    missing = [n for n, p in expected.items() if p.required and n not in found]
    unknown = sorted(n for n in found if n not in expected and not ignorable(n))
    unexpected = unknown if strict else []
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
    return unknown


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

    def __init__(self, model_dir, aliases: Optional[Mapping[str, str]] = None):
        """`aliases` maps a stored name to the name the model knows the tensor by; a
        tensor stored under its own name wins over one stored under an alias."""
        self.dir = Path(model_dir)
        paths = sorted(self.dir.glob("*.safetensors"))
        if not paths:
            raise FileNotFoundError(f"no *.safetensors file in {self.dir}")
        self.files: List[SafetensorsFile] = [SafetensorsFile(p) for p in paths]
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        self._where: Dict[str, Tuple[SafetensorsFile, str]] = {}
        aliases = dict(aliases or {})
        for direct in (True, False):
            for f in self.files:
                for n, meta in f.entries.items():
                    if (n not in aliases) != direct:
                        continue
                    name = n if direct else aliases[n]
                    if not direct and name in self.entries:
                        name = n                       # both are stored: the alias is one tensor too many
                    self.entries[name] = meta
                    self._where[name] = (f, n)

    def tensor(self, name: str) -> torch.Tensor:
        f, stored = self._where[name]
        return f.tensor(stored)

    def close(self) -> None:
        for f in self.files:
            f.close()


def _is_rotary_table(name: str) -> bool:
    return name.endswith("rotary_emb.inv_freq")


def _note(msg: str) -> None:
    print(f"[litinfer_amd] {msg}", file=sys.stderr, flush=True)


class TensorSource:
    """What `load_params` of a part is given: called with a tensor's name it returns
    the stored tensor on the CPU, or None for an optional tensor that is absent;
    `note(text)` reports a decision the part took about its tensors in one line."""

    def __init__(self, fetch: Callable[[str], Optional[torch.Tensor]], note: Callable[[str], None] = _note):
        self._fetch, self._note = fetch, note

    def __call__(self, name: str) -> Optional[torch.Tensor]:
        return self._fetch(name)

    def note(self, text: str) -> None:
        self._note(text)


def load_into(model, model_dir, aliases: Optional[Mapping[str, str]] = None, strict: bool = False,
              note: Callable[[str], None] = _note) -> List[str]:
    """Check the folder against `model.expected_params()` and hand each part its
    tensors (`model.load_params(get)`, where get(name) returns the stored tensor
    on the CPU or None for an optional tensor that is absent).  Returns the names
    of the stored tensors that the model does not use; they are reported through
    `note` in one line, or, when `strict`, are part of the error."""
    ckpt = CheckpointFolder(model_dir, aliases)
    try:
        expected = model.expected_params()
        unused = check_entries(expected, ckpt.entries, _is_rotary_table, strict=strict)
        if unused:
            shown = ", ".join(unused[:8]) + (f", ... and {len(unused) - 8} more" if len(unused) > 8 else "")
            note(f"{len(unused)} stored tensor(s) are not used by {model.spec.architecture}: {shown}")

        fetched = set()

        def get(name: str):
            if name not in ckpt.entries:
                return None
            if not expected[name].integer:
                fetched.add(ckpt.entries[name][0])
            return stored_precision(ckpt.tensor(name), expected[name].integer)

        rounded = getattr(getattr(model, "rt", None), "rounded", None)
        before = sum(rounded.values()) if rounded is not None else 0
        model.load_params(TensorSource(get, note))
        if rounded is not None and sum(rounded.values()) > before:
            stored = ", ".join(sorted(fetched - {"BF16"}))
            note(f"{sum(rounded.values()) - before} matrices stored as {stored} were rounded once (to nearest even) to "
                 f"bfloat16, the engine's dtype; keep_stored_precision=True keeps them in 32-bit")
        return unused
    finally:
        ckpt.close()
