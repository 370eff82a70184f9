"""Python side of the benchmark's measuring kernels (csrc/probe.hip): a kernel that only
reads, one that copies, a loop of bfloat16 MFMAs and a loop of float32 FMAs on registers.
Nothing on the product path uses them."""
from __future__ import annotations

from ctypes import c_int, c_long, c_void_p

import torch

from . import build

_fns = {}


def _fn(name, argtypes):
    f = _fns.get(name)
    if f is None:
        f = getattr(build.load("probe"), name)
        f.argtypes, f.restype = argtypes + [c_void_p], c_int
        _fns[name] = f
    return f


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


_sinks = {}


def _sink(device) -> torch.Tensor:
    if device not in _sinks:
        _sinks[device] = torch.zeros(64, dtype=torch.float32, device=device)
    return _sinks[device]


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: the probe library refused the call (code {rc})")


def _bytes_of(t: torch.Tensor) -> int:
    if not (t.is_cuda and t.is_contiguous() and t.data_ptr() % 16 == 0):
        raise ValueError("probe: needs a contiguous GPU tensor that starts on 16 bytes")
    return t.numel() * t.element_size()


def read(src: torch.Tensor, blocks: int = 256 * 16) -> None:
    """Read every byte of src once."""
    _check(_fn("li_probe_read", [c_void_p, c_long, c_void_p, c_int])(
        src.data_ptr(), _bytes_of(src), _sink(src.device).data_ptr(), blocks, _stream()), "probe.read")


def copy(src: torch.Tensor, dst: torch.Tensor, blocks: int = 256 * 16) -> None:
    if _bytes_of(dst) != _bytes_of(src):
        raise ValueError("probe.copy: src and dst differ in size")
    _check(_fn("li_probe_copy", [c_void_p, c_void_p, c_long, c_int])(
        src.data_ptr(), dst.data_ptr(), _bytes_of(src), blocks, _stream()), "probe.copy")


def mfma(blocks: int, iters: int, device="cuda:0") -> None:
    _check(_fn("li_probe_mfma", [c_void_p, c_int, c_int])(_sink(torch.device(device)).data_ptr(), blocks, iters, _stream()),
           "probe.mfma")


def mfma_flops(blocks: int, iters: int) -> float:
    return blocks * 4.0 * iters * 4 * 2 * 32 * 32 * 16


def fma(blocks: int, iters: int, device="cuda:0") -> None:
    _check(_fn("li_probe_fma", [c_void_p, c_int, c_int])(_sink(torch.device(device)).data_ptr(), blocks, iters, _stream()),
           "probe.fma")


def fma_flops(blocks: int, iters: int) -> float:
    return blocks * 256.0 * iters * 8 * 2
