"""Python side of the HIP kernels: argument checks and the ctypes calls.

Every function checks on the host that devices, dtypes, shapes and strides are
what its kernel and launch assume, because a kernel that reads out of bounds
can take the GPU down.  There is no fallback: on a tensor that is not on the
GPU, or without the built library, a call raises.
"""
from __future__ import annotations

import ctypes
import math
from ctypes import c_float, c_int, c_long, c_void_p
from typing import Dict, Optional

import numpy as np
import torch

from . import build
from ..utils.profiler import profiler

float32 = torch.float32
bfloat16 = torch.bfloat16

_DT = {torch.float32: 0, torch.bfloat16: 1}
MAX_HEAD_DIM = 256

P, I, F, L = c_void_p, c_int, c_float, c_long
_SIGNATURES = {
    "elementwise": {
        "li_embedding": [P, P, P, P, I, P, I, I, I],
        "li_rmsnorm": [P, I, P, F, P, I, I, I],
        "li_gather_rows": [P, P, P, I, I],
        "li_cast": [P, I, P, I, L],
        "li_swiglu": [P, P, I, I, I],
        "li_rope_table": [P, F, I, P, P, I],
        "li_rope_apply": [P, I, I, I, I, I, P, P, I],
        "li_kv_store": [P, I, I, I, I, I, P, P, P, I, I, I],
        "li_rope_kv_store": [P, I, I, I, I, I, I, P, P, P, P, P, I, I, I],
    },
    "gemm": {
        "li_linear": [P, P, P, P, I, I, I, I, I, I, P, L],
        "li_linear_skinny": [P, P, P, P, I, I, I, I, I, I],
        "li_linear_swiglu": [P, P, P, I, I, I, P, I, F],
        "li_linear_swiglu_f32": [P, P, P, I, I, I],
        "li_linear_residual_norm": [P, P, P, P, I, I, I, P, P, P],
        "li_linear_then_norm": [P, P, P, P, I, I, I, P, L, P, F, P, I],
        "li_linear_rope_store": [P, P, P, P, I, I, P, P, P, P, P, I, I, I, I, I, P, I, F],
        "li_linear_rope_store_parts": [P, P, P, P, I, I, P, P, P, P, P, I, I, I, I, I, P, L],
    },
    "attention": {
        "li_paged_attention": [P, I, P, P, P, I, P, I, P, P, P, P, P, I, I, I, I, I, I, I, I, I, I, F],
        "li_paged_attention_prefill": [P, I, P, P, P, P, I, P, I, P, P, P, I, I, I, I, I, I, F, I, P, P, P, I],
        "li_paged_attention_prefill_f32": [P, I, P, P, P, P, I, P, I, P, P, P, I, I, I, I, I, I, F],
        "li_paged_attention_decode": [P, I, P, P, P, I, P, I, P, I, P, P, P, P, P, P, I, I, I, I, I, I, F, I, I, P, P],
        "li_decode_run_keys": [P, I, P, P, P, P, I, I, I, I, I, I, I, P],
    },
    "sampling": {
        "li_argmax_rows": [P, P, P, P, I, I],
        "li_sample_rows": [P, P, P, P, P, P, I, I, P, L],
        "li_sample_prepare": [P, I, P, I, P, P, P, P],
    },
}
_fn_cache = {}


def _fn(module: str, name: str):
    key = (module, name)
    f = _fn_cache.get(key)
    if f is None:
        lib = build.load(module)
        f = getattr(lib, name)
        f.argtypes = _SIGNATURES[module][name] + [c_void_p]      # + stream
        f.restype = c_int
        _fn_cache[key] = f
    return f


def _work_bytes(m: int, n: int, k: int, dtype: int) -> int:
    f = _fn_cache.get(("gemm", "li_linear_work_bytes"))
    if f is None:
        f = build.load("gemm").li_linear_work_bytes
        f.argtypes, f.restype = [c_int, c_int, c_int, c_int], c_long
        _fn_cache[("gemm", "li_linear_work_bytes")] = f
    return int(f(m, n, k, dtype))


def _sample_scratch_floats(n: int, v: int) -> int:
    f = _fn_cache.get(("sampling", "li_sample_rows_scratch_floats"))
    if f is None:
        f = build.load("sampling").li_sample_rows_scratch_floats
        f.argtypes, f.restype = [c_int, c_int], c_long
        _fn_cache[("sampling", "li_sample_rows_scratch_floats")] = f
    return int(f(n, v))


PREFILL_RUNS_MAX_BYTES = 1 << 30       # room that the runs of a prompt portion's keys may take in the workspace


def _prefill_runs(host_q_len, host_ctx_len, nh: int, nkv: int, dh: int, max_blocks: int, window: int, tokens: int) -> int:
    """How many runs the library cuts the keys of a prompt portion's tiles into (the batch's segments as
    int32 arrays in host memory)."""
    f = _fn_cache.get(("attention", "li_paged_attention_prefill_runs"))
    if f is None:
        f = build.load("attention").li_paged_attention_prefill_runs
        f.argtypes, f.restype = [c_int, c_void_p, c_void_p] + [c_int] * 6 + [c_long], c_int
        _fn_cache[("attention", "li_paged_attention_prefill_runs")] = f
    if host_q_len is None or host_ctx_len is None or host_q_len.dtype != "int32" or host_ctx_len.dtype != "int32":
        return 1
    return int(f(len(host_q_len), host_q_len.ctypes.data, host_ctx_len.ctypes.data, nh, nkv, dh, max_blocks,
                 int(window), tokens, PREFILL_RUNS_MAX_BYTES))


# the current stream's handle without the stream object around it (an op is called some hundred times a
# step, and the object's way through torch's Python layers took a quarter of a step's host time)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    if _raw_stream is not None and _get_device is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


def _run(module: str, name: str, *args) -> None:
    if profiler.enabled:
        rc = []
        profiler.timed(name[3:], lambda: rc.append(_fn(module, name)(*args, _stream())), torch.cuda.synchronize)
        rc = rc[0]
    else:
        rc = _fn(module, name)(*args, _stream())
    if rc != 0:
        raise RuntimeError(f"{name}: the kernel library refused the call (code {rc}): "
                           f"{_ERRORS.get(rc, 'unknown')}")


_ERRORS = {1: "unsupported dtype combination", 2: "unsupported size", 3: "launch failed"}


def require_gpu(device) -> None:
    if not torch.cuda.is_available():
        raise RuntimeError("litinfer_amd runs on an AMD GPU through its HIP kernels; "
                           "no GPU is visible and there is no CPU path")


def _gpu(*ts) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("kernel call on a tensor that is not on the GPU "
                               "(there is no CPU path)")


def _chk(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _rows_ok(t: torch.Tensor) -> bool:
    return t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1]


def check_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Sizes the attention and position kernels take; anything else is refused
    here, when the model is built."""
    # (the texts are made only when they are needed: these checks run with every call of an op)
    if not (num_heads > 0 and num_kv_heads > 0 and num_heads % num_kv_heads == 0):
        _chk(False, f"attention: {num_heads} heads and {num_kv_heads} kv heads: the first must be a "
                    f"multiple of the second")
    if not (head_dim % 2 == 0 and 2 <= head_dim <= MAX_HEAD_DIM):
        _chk(False, f"attention: head size {head_dim} is not supported (even, at most {MAX_HEAD_DIM})")


# ---------------------------------------------------------------- elementwise
def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor,
              id_src: Optional[torch.Tensor] = None, feedback: Optional[torch.Tensor] = None) -> None:
    """out[t, :] = table[id(t), :] as float32 with id(t) = ids[t], or
    feedback[id_src[t]] where id_src is given and id_src[t] >= 0 (a token chosen
    on the device that the host has not seen yet).  Ids given by the host must
    already be inside the table (the step checks them); an id outside it (one
    that the device chose) gives a row of zeros, never a read outside the table."""
    _gpu(ids, table, out, id_src, feedback)
    t, h = out.shape
    _chk(ids.dtype is torch.int32 and ids.numel() == t and ids.is_contiguous(), "embedding: ids")
    _chk(table.dim() == 2 and table.shape[1] == h and table.is_contiguous() and table.dtype in _DT,
         "embedding: table")
    _chk(out.dtype is torch.float32 and out.is_contiguous(), "embedding: out must be float32")
    _chk(id_src is None or (feedback is not None and id_src.dtype is torch.int32 and id_src.numel() == t
                            and id_src.is_contiguous() and feedback.dtype is torch.int32
                            and feedback.is_contiguous()), "embedding: id_src / feedback")
    if t:
        _run("elementwise", "li_embedding", ids.data_ptr(), 0 if id_src is None else id_src.data_ptr(),
             0 if id_src is None else feedback.data_ptr(), table.data_ptr(), _DT[table.dtype],
             out.data_ptr(), t, h, table.shape[0])


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    _gpu(x, weight, out)
    _chk(x.dim() == 2 and x.shape == out.shape and x.is_contiguous() and out.is_contiguous(),
         "rmsnorm: x and out must be contiguous [T, H] of one shape")
    _chk(x.dtype in _DT and out.dtype in _DT, "rmsnorm: dtype")
    _chk(weight.dtype is torch.float32 and weight.numel() == x.shape[1] and weight.is_contiguous(),
         "rmsnorm: weight must be float32 [H]")
    if x.shape[0]:
        _run("elementwise", "li_rmsnorm", x.data_ptr(), _DT[x.dtype], weight.data_ptr(), float(eps),
             out.data_ptr(), _DT[out.dtype], x.shape[0], x.shape[1])


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    """out[i, :] = x[rows[i], :]; rows must be valid row numbers of x."""
    _gpu(x, rows, out)
    _chk(x.dtype is torch.float32 and out.dtype is torch.float32 and x.is_contiguous()
         and out.is_contiguous() and x.dim() == 2 and out.dim() == 2 and x.shape[1] == out.shape[1],
         "gather_rows: x, out")
    _chk(rows.dtype is torch.int32 and rows.numel() == out.shape[0] and rows.is_contiguous(),
         "gather_rows: rows")
    if out.shape[0]:
        _run("elementwise", "li_gather_rows", x.data_ptr(), rows.data_ptr(), out.data_ptr(),
             out.shape[0], x.shape[1])


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _gpu(src, dst)
    _chk(src.numel() == dst.numel() and src.is_contiguous() and dst.is_contiguous()
         and src.dtype in _DT and dst.dtype in _DT, "cast: src, dst")
    if src.numel():
        _run("elementwise", "li_cast", src.data_ptr(), _DT[src.dtype], dst.data_ptr(), _DT[dst.dtype],
             src.numel())


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, i] = up * gate / (1 + exp(-gate)) with gate = gate_up[t, i],
    up = gate_up[t, I + i]."""
    _gpu(gate_up, out)
    t, inter = out.shape
    _chk(gate_up.shape == (t, 2 * inter) and gate_up.is_contiguous() and out.is_contiguous()
         and gate_up.dtype is out.dtype and out.dtype in _DT, "swiglu: gate_up [T, 2I], out [T, I]")
    if t:
        _run("elementwise", "li_swiglu", gate_up.data_ptr(), out.data_ptr(), _DT[out.dtype], t, inter)


def rope_table(positions: torch.Tensor, theta: float, rotary_dim: int, cos: torch.Tensor,
               sin: torch.Tensor) -> None:
    """cos/sin [T, rotary_dim/2] of angle = float(pos) / theta^(2j/rotary_dim), in float32."""
    _gpu(positions, cos, sin)
    t = positions.numel()
    _chk(positions.dtype is torch.int32 and positions.is_contiguous(), "rope_table: positions")
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and cos.is_contiguous()
         and sin.is_contiguous() and cos.dtype is torch.float32 and sin.dtype is torch.float32,
         "rope_table: cos, sin")
    if t:
        _run("elementwise", "li_rope_table", positions.data_ptr(), float(theta), rotary_dim,
             cos.data_ptr(), sin.data_ptr(), t)


def _check_qkv(qkv, heads_total, head_dim):
    _chk(_rows_ok(qkv) and qkv.dtype in _DT and qkv.shape[1] >= heads_total * head_dim,
         "qkv: needs rows of at least heads*head_dim elements")


def rope_apply(qkv: torch.Tensor, n_heads: int, head_dim: int, rotary_dim: int, cos: torch.Tensor,
               sin: torch.Tensor) -> None:
    """Rotate heads 0..n_heads-1 of every row of qkv in place (half-split pairs)."""
    _gpu(qkv, cos, sin)
    _check_qkv(qkv, n_heads, head_dim)
    t = qkv.shape[0]
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and rotary_dim <= head_dim,
         "rope_apply: tables")
    if t:
        _run("elementwise", "li_rope_apply", qkv.data_ptr(), _DT[qkv.dtype], qkv.stride(0), n_heads,
             head_dim, rotary_dim, cos.data_ptr(), sin.data_ptr(), t)


def _check_cache(k, v, nkv, dh, page_size, dtype):
    _chk(k.shape == v.shape and k.dim() == 4 and k.shape[1:] == (nkv, page_size, dh)
         and k.is_contiguous() and v.is_contiguous() and k.dtype is dtype and v.dtype is dtype,
         "kv cache: expected contiguous [pages, kv_heads, page_size, head_dim] of the activation dtype")


def kv_store(qkv: torch.Tensor, nh: int, nkv: int, dh: int, slot_map: torch.Tensor, k: torch.Tensor,
             v: torch.Tensor, page_size: int) -> None:
    """Write the key and value heads of every row of qkv (columns nh*dh.. and
    (nh+nkv)*dh..) to the page slot slot_map[t] = page*page_size + offset."""
    _gpu(qkv, slot_map, k, v)
    _check_qkv(qkv, nh + 2 * nkv, dh)
    _check_cache(k, v, nkv, dh, page_size, qkv.dtype)
    t = qkv.shape[0]
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == t and slot_map.is_contiguous(),
         "kv_store: slot_map")
    if t:
        _run("elementwise", "li_kv_store", qkv.data_ptr(), _DT[qkv.dtype], qkv.stride(0), nh, nkv, dh,
             slot_map.data_ptr(), k.data_ptr(), v.data_ptr(), page_size, k.shape[0], t)


def rope_kv_store(qkv: torch.Tensor, nh: int, nkv: int, dh: int, rotary_dim: int, cos: torch.Tensor,
                  sin: torch.Tensor, slot_map: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  page_size: int) -> None:
    """Fused: rotate the query heads in place, rotate the key heads and write
    them, and copy the value heads, to the pages."""
    _gpu(qkv, cos, sin, slot_map, k, v)
    _check_qkv(qkv, nh + 2 * nkv, dh)
    _check_cache(k, v, nkv, dh, page_size, qkv.dtype)
    t = qkv.shape[0]
    _chk(cos.shape == (t, rotary_dim // 2) and sin.shape == cos.shape and rotary_dim <= dh
         and cos.dtype is torch.float32, "rope_kv_store: tables")
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == t and slot_map.is_contiguous(),
         "rope_kv_store: slot_map")
    if t:
        _run("elementwise", "li_rope_kv_store", qkv.data_ptr(), _DT[qkv.dtype], qkv.stride(0), nh, nkv,
             dh, rotary_dim, cos.data_ptr(), sin.data_ptr(), slot_map.data_ptr(), k.data_ptr(),
             v.data_ptr(), page_size, k.shape[0], t)


# ---------------------------------------------------------------------- gemm
SKINNY_MAX_ROWS = 64
SPLITK_MAX_PARTS = 8


def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           accumulate: bool = False, ws=None) -> None:
    """out = x w^T + bias, or out += x w^T + bias when `accumulate`.
    x [M, K] and w [N, K] of one dtype (float32 or bfloat16); out [M, N] of that
    dtype or float32; accumulation of the product is float32.  `ws` lends the
    memory for partial sums where the kernel cuts K into parts (17 rows and more
    against a matrix of few columns); without it
    such a product takes a slower kernel."""
    _gpu(x, w, bias, out)
    _chk(x.dim() == 2 and w.dim() == 2 and out.dim() == 2, "linear: needs matrices")
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape[1] == k and out.shape == (m, n)):
        _chk(False, f"linear: shapes x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear: contiguous operands")
    if not (x.dtype is w.dtype and x.dtype in _DT):
        _chk(False, f"linear: x is {x.dtype}, w is {w.dtype}")
    _chk(out.dtype is x.dtype or out.dtype is torch.float32, "linear: out dtype")
    _chk(not accumulate or out.dtype is torch.float32, "linear: accumulation needs a float32 out")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear: bias must be float32 [N]")
    if m:
        work, work_bytes = 0, 0
        if ws is not None and x.dtype is torch.bfloat16 and not few_rows_preferred(m, n, k):
            # few rows over a long k and few columns: the library cuts k into parts if it is lent room for their sums
            need = _work_bytes(m, n, k, _DT[x.dtype])
            if need:
                if m <= SKINNY_MAX_ROWS:            # one size for all row counts of a decode batch: the buffer does not move
                    need = max(need, SPLITK_MAX_PARTS * SKINNY_MAX_ROWS * n * 4)
                buf = ws.buffer("gemm.parts", (need // 4,), torch.float32)
                work, work_bytes = buf.data_ptr(), buf.numel() * 4
        _run("gemm", "li_linear", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
             out.data_ptr(), m, n, k, _DT[x.dtype], _DT[out.dtype], int(bool(accumulate)), work, work_bytes)



def linear_row_tile(dtype: torch.dtype) -> int:
    """Rows of the smallest tile that `linear` cuts a product of many rows of this dtype into (the
    kernel library says): a few rows more than a multiple of it cost a whole tile more."""
    f = _fn_cache.get(("gemm", "li_linear_row_tile"))
    if f is None:
        f = build.load("gemm").li_linear_row_tile
        f.argtypes, f.restype = [c_int], c_int
        _fn_cache[("gemm", "li_linear_row_tile")] = f
    return int(f(_DT[dtype]))


def skinny_takes(m: int, k: int, w_dtype: torch.dtype) -> bool:
    """Whether `linear_skinny` takes a product of m rows over k with such a matrix."""
    return w_dtype is torch.bfloat16 and k % 8 == 0 and 0 < m <= SKINNY_MAX_ROWS


def linear_skinny(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  accumulate: bool = False, swiglu: bool = False) -> None:
    """The product for few rows (decoding).  swiglu: w is [gate; up] (2N rows)
    and out[m, n] = up * gate / (1 + exp(-gate)), the activation fused into the
    product's epilogue."""
    _gpu(x, w, bias, out)
    m, k = x.shape
    n = out.shape[1]
    _chk(skinny_takes(m, k, w.dtype), "linear_skinny: sizes or dtype not taken")
    _chk(w.shape == ((2 * n if swiglu else n), k) and out.shape[0] == m, "linear_skinny: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_skinny: contiguous operands")
    _chk(x.dtype is torch.bfloat16, "linear_skinny: x must be bfloat16")
    _chk(out.dtype in _DT and (not accumulate or out.dtype is torch.float32), "linear_skinny: out dtype")
    _chk(not swiglu or (bias is None and not accumulate and out.dtype is torch.bfloat16),
         "linear_skinny: swiglu takes no bias and no accumulation and writes bfloat16")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_skinny: bias must be float32 [N]")
    _run("gemm", "li_linear_skinny", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
         out.data_ptr(), m, n, k, _DT[out.dtype], int(bool(accumulate)), int(bool(swiglu)))


def swiglu_takes(m: int, k: int, w_dtype: torch.dtype) -> bool:
    """Whether `linear_swiglu` takes a product of m rows over k with such a matrix (float32: the few rows of
    a decoding step)."""
    if w_dtype is torch.float32:
        # (more rows: a block's share of x grows with them while its gate and up columns stay 16 each; the
        # product without the activation takes wider blocks there)
        return 0 < m <= 16 and k % 4 == 0
    return w_dtype is torch.bfloat16 and m > 0 and (k % 8 == 0 if m <= SKINNY_MAX_ROWS else k % 64 == 0)


# An RMS norm between two products of few rows (a decoding step), without a pass of its own: the
# product before it, which adds to the float32 sum, also writes the sum times the norm's weights in
# bfloat16 and each block's share of the rows' sums of squares (`linear_residual_norm`); the product
# after it multiplies those rows and scales each row's result by the norm's factor (`row_scale` of
# `linear_swiglu` and `linear_rope_store`).
RESIDUAL_NORM_MAX_ROWS = 32
RESIDUAL_NORM_MAX_PARTS = 512
# The few-row kernels with their fused epilogues take up to 32 rows (two tiles of 16 a block); from 13 rows on
# the 64-row tiles with K in parts (and the kernels that add the parts up doing the norm, the rotation and the
# page write) are faster where the matrix is large, from 17 on also where it is of middling size.  Parts ask `few_rows_preferred` beside the `*_takes` of the few-row
# kernels; the kernel library holds the rule (its own entry points decide by it too).


def few_rows_preferred(m: int, n: int, k: int) -> bool:
    """Whether m rows against a matrix [n, k] should take the few-row kernels."""
    f = _fn_cache.get(("gemm", "li_few_rows_preferred"))
    if f is None:
        f = build.load("gemm").li_few_rows_preferred
        f.argtypes, f.restype = [c_int, c_long, c_long], c_int
        _fn_cache[("gemm", "li_few_rows_preferred")] = f
    return bool(f(int(m), int(n), int(k)))


class RowScale:
    """What the product after a fused RMS norm needs beside its rows: the shares of the rows' sums
    of squares [nparts * R] float32 (R = 16 for up to 16 rows, 32 above) and the norm's eps."""
    def __init__(self, sq_parts: torch.Tensor, nparts: int, eps: float):
        self.sq_parts, self.nparts, self.eps = sq_parts, int(nparts), float(eps)


def residual_norm_parts(n: int) -> int:
    """Blocks of `linear_residual_norm` over n columns, i.e. shares of a row's sum of squares (the
    library spreads a matrix of few columns evenly over the current device's compute units)."""
    f = _fn_cache.get(("gemm", "li_residual_norm_parts"))
    if f is None:
        f = build.load("gemm").li_residual_norm_parts
        f.argtypes, f.restype = [c_int], c_int
        _fn_cache[("gemm", "li_residual_norm_parts")] = f
    return int(f(int(n)))


def residual_norm_takes(m: int, n: int, k: int, w_dtype: torch.dtype) -> bool:
    return (w_dtype is torch.bfloat16 and 0 < m <= RESIDUAL_NORM_MAX_ROWS and k % 8 == 0
            and residual_norm_parts(n) <= RESIDUAL_NORM_MAX_PARTS)


def row_scale_rows(m: int) -> int:
    """Places a block's shares of the rows' sums of squares take: 16 for up to 16 rows, 32 above."""
    return 16 if m <= 16 else 32


def linear_residual_norm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                         gamma: torch.Tensor, xg: torch.Tensor, sq_parts: torch.Tensor) -> int:
    """out += x w^T + bias (float32); xg = bfloat16(gamma * out); sq_parts[p * R + m] = block p's
    share of sum_n out[m, n]^2 (R = `row_scale_rows(m)`).  Returns the number of blocks p."""
    _gpu(x, w, bias, out, gamma, xg, sq_parts)
    m, k = x.shape
    n = w.shape[0]
    _chk(residual_norm_takes(m, n, k, w.dtype), "linear_residual_norm: sizes or dtype not taken")
    _chk(x.dtype is torch.bfloat16 and w.shape == (n, k) and x.is_contiguous() and w.is_contiguous(),
         "linear_residual_norm: x and w must be contiguous bfloat16 [M, K] and [N, K]")
    _chk(out.dtype is torch.float32 and out.shape == (m, n) and out.is_contiguous(), "linear_residual_norm: out must be float32 [M, N]")
    _chk(xg.dtype is torch.bfloat16 and xg.shape == (m, n) and xg.is_contiguous(), "linear_residual_norm: xg must be bfloat16 [M, N]")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_residual_norm: bias must be float32 [N]")
    _chk(gamma.dtype is torch.float32 and gamma.shape == (n,) and gamma.is_contiguous(), "linear_residual_norm: gamma must be float32 [N]")
    parts = residual_norm_parts(n)
    _chk(sq_parts.dtype is torch.float32 and sq_parts.is_contiguous() and sq_parts.numel() >= parts * row_scale_rows(m),
         "linear_residual_norm: sq_parts must be float32 with 16 places a block (32 above 16 rows)")
    _run("gemm", "li_linear_residual_norm", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
         out.data_ptr(), m, n, k, gamma.data_ptr(), xg.data_ptr(), sq_parts.data_ptr())
    return parts


def linear_then_norm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                     gamma: torch.Tensor, eps: float, xn: torch.Tensor, ws) -> bool:
    """out += x w^T + bias (float32) and xn = gamma * out / sqrt(mean(out^2) + eps), in the kernel
    that adds up the parts of a product cut along K.  Returns False, having done nothing, where
    `linear` would not cut this product (then multiply and norm in two calls)."""
    _gpu(x, w, bias, out, gamma, xn)
    if ws is None or x.dtype is not torch.bfloat16 or w.dtype is not torch.bfloat16:
        return False
    _chk(x.dim() == 2 and w.dim() == 2, "linear_then_norm: needs matrices")
    m, k = x.shape
    n = w.shape[0]
    need = _work_bytes(m, n, k, _DT[x.dtype])
    if not need:
        return False
    _chk(w.shape == (n, k) and x.is_contiguous() and w.is_contiguous(), "linear_then_norm: contiguous [M, K] and [N, K]")
    _chk(out.dtype is torch.float32 and out.shape == (m, n) and out.is_contiguous(), "linear_then_norm: out must be float32 [M, N]")
    _chk(xn.dtype in _DT and xn.shape == (m, n) and xn.is_contiguous(), "linear_then_norm: xn must be [M, N]")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_then_norm: bias must be float32 [N]")
    _chk(gamma.dtype is torch.float32 and gamma.shape == (n,) and gamma.is_contiguous() and eps >= 0,
         "linear_then_norm: gamma must be float32 [N], eps not negative")
    if m <= SKINNY_MAX_ROWS:                # one size for all row counts of a decode batch: the buffer does not move
        need = max(need, SPLITK_MAX_PARTS * SKINNY_MAX_ROWS * n * 4)
    buf = ws.buffer("gemm.parts", (need // 4,), torch.float32)
    rc = _fn("gemm", "li_linear_then_norm")(x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
                                             out.data_ptr(), m, n, k, buf.data_ptr(), buf.numel() * 4, gamma.data_ptr(),
                                             float(eps), xn.data_ptr(), _DT[xn.dtype], _stream())
    if rc == -1:
        return False
    if rc != 0:
        raise RuntimeError(f"li_linear_then_norm: the kernel library refused the call (code {rc}): {_ERRORS.get(rc, 'unknown')}")
    return True


def _check_row_scale(what: str, m: int, row_scale: Optional[RowScale]):
    if row_scale is None:
        return 0, 0, 0.0
    _gpu(row_scale.sq_parts)
    _chk(0 < m <= RESIDUAL_NORM_MAX_ROWS, f"{what}: a row scale goes with up to {RESIDUAL_NORM_MAX_ROWS} rows")
    _chk(0 < row_scale.nparts <= RESIDUAL_NORM_MAX_PARTS and row_scale.eps >= 0, f"{what}: row scale out of range")
    _chk(row_scale.sq_parts.dtype is torch.float32 and row_scale.sq_parts.is_contiguous()
         and row_scale.sq_parts.numel() >= row_scale.nparts * row_scale_rows(m),
         f"{what}: the row scale's parts must be float32 [nparts * {row_scale_rows(m)}]")
    return row_scale.sq_parts.data_ptr(), row_scale.nparts, row_scale.eps


def linear_swiglu(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, row_scale: Optional[RowScale] = None) -> None:
    """out[m, n] = up * gate / (1 + exp(-gate)) with [gate, up] = x w^T, w = [gate; up]
    (2 N rows): the activation in the product's epilogue, from the product's float32 sums.
    With `row_scale`, x is the xg of `linear_residual_norm` and the result is that of the norm."""
    _gpu(x, w, out)
    _chk(x.dim() == 2 and w.dim() == 2 and out.dim() == 2, "linear_swiglu: needs matrices")
    m, k = x.shape
    n = out.shape[1]
    _chk(swiglu_takes(m, k, w.dtype) or (w.dtype is torch.float32 and 0 < m <= SKINNY_MAX_ROWS and k % 4 == 0),
         "linear_swiglu: sizes or dtype not taken")
    _chk(w.shape == (2 * n, k) and out.shape[0] == m, "linear_swiglu: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_swiglu: contiguous operands")
    if w.dtype is torch.float32:
        _chk(x.dtype is torch.float32 and out.dtype is torch.float32 and row_scale is None,
             "linear_swiglu: float32 w goes with float32 x and out, and no row scale")
        _chk(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "linear_swiglu: operands must start on 16 bytes")
        _run("gemm", "li_linear_swiglu_f32", x.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k)
        return
    _chk(x.dtype is torch.bfloat16 and out.dtype is torch.bfloat16, "linear_swiglu: x and out must be bfloat16")
    _run("gemm", "li_linear_swiglu", x.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k,
         *_check_row_scale("linear_swiglu", m, row_scale))


ROPE_STORE_MAX_ROWS = 32


def rope_store_takes(m: int, k: int, w_dtype: torch.dtype, dh: int, rotary_dim: int) -> bool:
    """Whether `linear_rope_store` takes the packed projection of m rows over k."""
    return (w_dtype is torch.bfloat16 and 0 < m <= ROPE_STORE_MAX_ROWS and k % 8 == 0
            and dh % 16 == 0 and rotary_dim == dh)


def linear_rope_store(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                      nh: int, nkv: int, dh: int, cos: torch.Tensor, sin: torch.Tensor,
                      slot_map: torch.Tensor, k: torch.Tensor, v: torch.Tensor, page_size: int,
                      row_scale: Optional[RowScale] = None) -> None:
    """Fused for a decoding step: out = x w^T + bias with w the packed [q; k; v]
    projection, query and key heads rotated (half-split pairs, the whole head) by
    the rows' angles, keys and values written into their page slots.  out holds
    the rotated queries and keys and the values, as after the separate kernels.
    With `row_scale`, x is the xg of `linear_residual_norm` and the result is that of the norm."""
    _gpu(x, w, bias, out, cos, sin, slot_map, k, v)
    m, kk = x.shape
    n = (nh + 2 * nkv) * dh
    _chk(rope_store_takes(m, kk, w.dtype, dh, 2 * cos.shape[1]), "linear_rope_store: sizes or dtype not taken")
    _chk(w.shape == (n, kk) and out.shape == (m, n), "linear_rope_store: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_rope_store: contiguous operands")
    _chk(x.dtype is torch.bfloat16 and out.dtype is torch.bfloat16, "linear_rope_store: x and out must be bfloat16")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_rope_store: bias must be float32 [N]")
    _check_cache(k, v, nkv, dh, page_size, out.dtype)
    _chk(cos.shape == (m, dh // 2) and sin.shape == cos.shape and cos.dtype is torch.float32
         and sin.dtype is torch.float32 and cos.is_contiguous() and sin.is_contiguous(), "linear_rope_store: tables")
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == m and slot_map.is_contiguous(),
         "linear_rope_store: slot_map")
    _run("gemm", "li_linear_rope_store", x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(),
         out.data_ptr(), m, kk, cos.data_ptr(), sin.data_ptr(), slot_map.data_ptr(), k.data_ptr(), v.data_ptr(),
         nh, nkv, dh, page_size, k.shape[0], *_check_row_scale("linear_rope_store", m, row_scale))


def linear_rope_store_parts(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                            nh: int, nkv: int, dh: int, cos: torch.Tensor, sin: torch.Tensor,
                            slot_map: torch.Tensor, k: torch.Tensor, v: torch.Tensor, page_size: int, ws) -> bool:
    """The same result as `linear_rope_store` for the rows of a large decoding batch, where the
    packed projection is cut along K anyway: the kernel that adds the parts up rotates and writes
    the pages.  Returns False, having done nothing, where `linear` would not cut this product."""
    _gpu(x, w, bias, out, cos, sin, slot_map, k, v)
    if ws is None or x.dtype is not torch.bfloat16 or w.dtype is not torch.bfloat16 or 2 * cos.shape[1] != dh:
        return False
    m, kk = x.shape
    n = (nh + 2 * nkv) * dh
    need = _work_bytes(m, n, kk, _DT[x.dtype])
    if not need:
        return False
    _chk(w.shape == (n, kk) and out.shape == (m, n), "linear_rope_store_parts: shapes do not fit")
    _chk(x.is_contiguous() and w.is_contiguous() and out.is_contiguous(), "linear_rope_store_parts: contiguous operands")
    _chk(out.dtype is torch.bfloat16, "linear_rope_store_parts: out must be bfloat16")
    _chk(bias is None or (bias.dtype is torch.float32 and bias.numel() == n and bias.is_contiguous()),
         "linear_rope_store_parts: bias must be float32 [N]")
    _check_cache(k, v, nkv, dh, page_size, out.dtype)
    _chk(cos.shape == (m, dh // 2) and sin.shape == cos.shape and cos.dtype is torch.float32
         and sin.dtype is torch.float32 and cos.is_contiguous() and sin.is_contiguous(), "linear_rope_store_parts: tables")
    _chk(slot_map.dtype is torch.int32 and slot_map.numel() == m and slot_map.is_contiguous(),
         "linear_rope_store_parts: slot_map")
    if m <= SKINNY_MAX_ROWS:                # one size for all row counts of a decode batch: the buffer does not move
        need = max(need, SPLITK_MAX_PARTS * SKINNY_MAX_ROWS * n * 4)
    buf = ws.buffer("gemm.parts", (need // 4,), torch.float32)
    rc = _fn("gemm", "li_linear_rope_store_parts")(
        x.data_ptr(), w.data_ptr(), 0 if bias is None else bias.data_ptr(), out.data_ptr(), m, kk,
        cos.data_ptr(), sin.data_ptr(), slot_map.data_ptr(), k.data_ptr(), v.data_ptr(), nh, nkv, dh, page_size,
        k.shape[0], buf.data_ptr(), buf.numel() * 4, _stream())
    if rc == -1:
        return False
    if rc != 0:
        raise RuntimeError(f"li_linear_rope_store_parts: the kernel library refused the call (code {rc}): {_ERRORS.get(rc, 'unknown')}")
    return True


# ----------------------------------------------------------------- attention
# waves that the split-key decode kernel on the matrix cores is cut into at least (where the keys allow):
# four a compute unit; more splits cost more in the merge than they gain (measured at 8 and 64 requests)
_DEC_WAVES = 1024
PREFILL_TILE_ROWS = 32       # queries of one segment that a block of the matrix-core kernel for portions takes
DECODE_MAX_SPLITS = 64       # the merge kernel keeps a weight per split
DECODE_TABLE_CAP = 1024      # pages of one split that the matrix-core decode kernel copies into LDS
DECODE_LIST_MAX_TOKENS = 4096    # single tokens whose runs the device lists (`decode_run_keys`)


_simds: Dict[int, int] = {}


def _simd_count(device: torch.device) -> int:
    """Waves of the decode kernel that run at one time: one on each SIMD, four SIMDs a compute unit."""
    i = device.index if device.index is not None else torch.cuda.current_device()
    if i not in _simds:
        _simds[i] = 4 * torch.cuda.get_device_properties(i).multi_processor_count
    return _simds[i]


DECODE_QUAD = 4              # runs of a token's keys that one block of the matrix-core decode kernel takes, one a wave
# measurements only: single-wave blocks and a merge kernel behind them, as before the blocks joined their runs
_decode_single_waves = False
# Share of the SIMDs that a step's waves must fill for the blocks of four waves (below).  Most batch sizes give a
# number of runs whose waves fill the SIMDs nearly, not wholly (17 requests x 2 kv heads x 28 runs = 952 of
# 1,024); asked for all of them, those took single-wave blocks and the merge kernel: 17 / 24 / 28 requests of
# 4,096 keys at the 1.5B head layout 23.5 / 29.4 / 31.5 us a layer against 21.8 / 26.9 / 29.9 with the blocks of
# four (7B layout, 28 requests: 53.6 against 50.0); from a half on the short contexts lose (17.0 against 16.0 us).
_DECODE_FILLS = 0.7


def decode_splits(pairs: int, keys: int, simds: int = _DEC_WAVES, quad: int = DECODE_QUAD) -> int:
    """Into how many runs the keys of a decoding token are cut.  Every (token, kv head) pair and
    run is one wave, and a SIMD holds one wave of this kernel: the waves go over the SIMDs in
    rounds, each as long as a run (plus a wave's start and end, about 24 keys' time), so the
    number of runs with the least rounds x run length is taken, a run being a multiple of 32
    keys and at least 128 where the keys allow; every run costs the join a little (4 keys' time).
    The runs come in blocks of `quad` waves (a block joins its runs itself), so their number is 1
    or a multiple of `quad`.  Few pairs: as many runs as fill the SIMDs once."""
    most = max(1, min(-(-keys // 128), DECODE_MAX_SPLITS))
    best, best_cost = 1, None
    for ns in [1] + list(range(quad, most + 1, quad)):
        run = (-(-keys // ns) + 31) & ~31
        cost = -(-pairs * ns // simds) * (run + 24) + 4 * ns
        if best_cost is None or cost < best_cost:
            best, best_cost = ns, cost
    return best


def _ragged_splits(nsplit: int, meta, window: int, quad: int = DECODE_QUAD) -> int:
    """More runs for the grid of a batch whose contexts differ: `nsplit` fits contexts that are all as
    long as the longest; with one run length for the batch (chosen on the device) the short ones fill
    few runs, and the same number of working waves needs the longest cut into more."""
    ql, cl = getattr(meta, "host_q_len", None), getattr(meta, "host_ctx_len", None)
    if ql is None or cl is None or nsplit >= DECODE_MAX_SPLITS:
        return nsplit
    keys = cl[ql == 1]
    if keys.size < 2:
        return nsplit
    if window > 0:
        keys = np.minimum(keys, window)
    ragged = float(keys.max()) * keys.size / max(float(keys.sum()), 1.0)
    if ragged < 1.15:
        return nsplit
    more = min(DECODE_MAX_SPLITS, int(math.ceil(nsplit * ragged * 1.25)))
    return min(DECODE_MAX_SPLITS, -(-more // quad) * quad)


def decode_run_keys(meta, token_list: Optional[torch.Tensor], n_tokens: int, page_size: int, window: int,
                    nkv: int, nsplit: int, simds: int, out: torch.Tensor, group: int = 1) -> None:
    """out[0] = the run length, in keys, for the split-key decode kernel over these single tokens
    (`token_list`, or the batch's first n_tokens tokens): the multiple of 32 with the least rounds of
    working waves over `simds` x (length + 24), between what the longest context needs to fit
    `nsplit` runs and what the block table's width would need.  out[1] = the number of runs with
    keys at that length, out[2 : 2 + n_tokens] = the runs of each token, then the runs themselves as
    token | run << 16.  With `group` > 1 the runs are taken `group` at a time (one block of the decode
    kernel): the list then holds the first run of every group, out[1] counts the groups, and a length's
    cost counts `group` waves a group.  At most 4,096 tokens."""
    _gpu(out, meta.ctx_len, token_list)
    _chk(0 < n_tokens <= DECODE_LIST_MAX_TOKENS, "decode_run_keys: too many tokens")
    _chk(out.dtype is torch.int32 and out.is_contiguous() and out.numel() >= 2 + n_tokens + n_tokens * nsplit,
         "decode_run_keys: out must be int32 [2 + tokens + tokens * nsplit]")
    _run("attention", "li_decode_run_keys", 0 if token_list is None else token_list.data_ptr(), n_tokens,
         meta.seg_of_token.data_ptr(), meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
         meta.max_blocks, page_size, int(window), nkv, nsplit, simds, int(group), out.data_ptr())


def decode_split_blocks(max_blocks: int, page_size: int, window: int, nsplit: int) -> int:
    """The most pages one of `nsplit` splits of the keys can touch, for block tables of
    `max_blocks` pages: the keys (at most the table's, or the window's) are cut into runs
    of a multiple of 32, and a run that begins anywhere in a page touches one page more
    than its length fills.  The kernel library computes the same bound and refuses a call
    beyond its table."""
    keys = max_blocks * page_size
    if 0 < window < keys:
        keys = window
    per = (-(-keys // nsplit) + 31) & ~31
    return (per + page_size - 2) // page_size + 1

def _decode_kernel_takes(dtype: torch.dtype, dh: int) -> bool:
    """The single-query kernel spreads a key's row over dh / (16 bytes) lanes, a power of two."""
    per = 8 if dtype is torch.bfloat16 else 4
    return dh % per == 0 and (dh // per) & (dh // per - 1) == 0 and dh // per <= 64


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, k: torch.Tensor, v: torch.Tensor, meta,
                    nh: int, nkv: int, dh: int, page_size: int, window: int, scale: float,
                    ws=None) -> None:
    """Causal grouped-query attention of the batch's queries (heads 0..nh-1 of
    qkv's rows) over the paged keys and values; out [T, nh*dh].  Query i of a
    segment stands at position ctx_len - q_len + i and sees the keys at
    positions <= its own and, with window > 0, closer than `window`.  Tokens of
    segments that bring one token go to the split-key decode kernel, the others
    to the kernel for portions.  `ws` lends the buffers for the splits' partial
    results."""
    _gpu(qkv, out, k, v, meta.block_table)
    check_attention_sizes(nh, nkv, dh)
    _check_qkv(qkv, nh, dh)
    _check_cache(k, v, nkv, dh, page_size, qkv.dtype)
    t = qkv.shape[0]
    _chk(out.shape == (t, nh * dh) and out.is_contiguous() and out.dtype is qkv.dtype, "attention: out")
    _chk(t == meta.num_tokens, "attention: batch metadata is of another batch")
    bt = meta.block_table
    _chk(bt.dtype is torch.int32 and bt.shape == (meta.num_segments, meta.max_blocks)
         and bt.is_contiguous(), "attention: block table")
    _chk(meta.max_blocks * page_size >= meta.max_ctx_len, "attention: block table too short")
    _chk(meta.num_single + meta.num_multi == t, "attention: token lists do not cover the batch")
    _chk(meta.num_single in (0, t) or (meta.single_tokens is not None and meta.multi_tokens is not None),
         "attention: a batch of single-token and longer segments needs their token lists (BatchNeeds.token_kinds)")
    if not t:
        return
    n_single, n_multi = meta.num_single, meta.num_multi
    if n_single and not _decode_kernel_takes(qkv.dtype, dh):
        n_single, n_multi = 0, t                      # every token through the general kernel
    if n_single:
        keys = min(meta.max_single_ctx, window) if window > 0 else meta.max_single_ctx
        # a head size of 64 or 128 (bfloat16, or float32 on the float32 matrix cores): one wave per split
        # on the matrix cores; else one block of four waves per split on the vector ALU
        mfma = dh in (64, 128)
        planned = 0
        if mfma:
            # (the kernel finds a key's page by a float32 product that is exact below 2^22)
            _chk(meta.max_blocks * page_size <= 1 << 21 and page_size <= 1 << 16,
                 f"attention: block tables of {meta.max_blocks} pages of {page_size} keys are beyond the decode "
                 f"kernel's {1 << 21} keys")
            # Blocks of four waves that join their runs themselves, or single-wave blocks and a merge kernel
            # behind them.  Four waves sit on ONE compute unit and the join is three trips to memory at the
            # kernel's end: it pays where one block holds all runs of a (token, kv head) (no join, no second
            # kernel: 64 requests at the 7B head layout 105 -> 96 us a layer), and where the waves fill the
            # chip anyway and the runs are not many or long (8 requests, 4,096 keys: 22.3 -> 21.6 us; 8
            # requests of the 1.5B layout with 64 short runs each: 17.3 -> 18.9 us, so not there).  Not for
            # contexts that differ (one run length for the batch and a list of the runs that have keys): a
            # token's runs then fill its last block of four only partly, and a block's waves end at different
            # times (64 requests with 16 to 4,600 keys, 7B head layout: 73.8 us against 82.7; 1.5B: 41.3 / 52.5).
            simds = _simd_count(qkv.device)
            quad = DECODE_QUAD
            planned = decode_splits(n_single * nkv, keys, simds, quad)
            nsplit = _ragged_splits(planned, meta, window)
            fills = n_single * nkv * nsplit >= _DECODE_FILLS * simds
            if (_decode_single_waves or nsplit > planned
                    or not (nsplit == DECODE_QUAD or (fills and (nsplit <= 32 or keys >= 8192)))):
                quad = 1
                planned = decode_splits(n_single * nkv, keys, simds, quad)
                nsplit = _ragged_splits(planned, meta, window, quad)
            # a split's pages must fit the kernel's copy of the block table
            while nsplit <= DECODE_MAX_SPLITS and decode_split_blocks(meta.max_blocks, page_size, window, nsplit) > DECODE_TABLE_CAP:
                nsplit += 1 if nsplit < quad else quad
            if 1 < nsplit < quad:
                nsplit = quad
            _chk(nsplit <= DECODE_MAX_SPLITS, f"attention: block tables of {meta.max_blocks} pages of {page_size} "
                                              f"are too long for the decode kernel")
        else:
            nsplit = max(1, min(-(-512 // (n_single * nkv)), -(-keys // 256), DECODE_MAX_SPLITS))
        acc = ml = None
        if nsplit > 1:
            shape_a, shape_m = (n_single, nh, nsplit, dh), (n_single, nh, nsplit, 2)
            if ws is not None:
                acc = ws.buffer("attn.part_acc", shape_a, torch.float32)
                ml = ws.buffer("attn.part_ml", shape_m, torch.float32)
            else:
                acc = torch.empty(shape_a, dtype=torch.float32, device=qkv.device)
                ml = torch.empty(shape_m, dtype=torch.float32, device=qkv.device)
        lst = meta.single_tokens if n_single < t else None
        run_keys = done = None
        if mfma and nsplit > DECODE_QUAD and quad > 1:
            # the blocks of a (token, kv head) count themselves here, and the last one joins their results
            # (zero before the first call; every call leaves it zero)
            done = (ws.buffer("attn.done", (n_single * nkv,), torch.int32, zero=True) if ws is not None
                    else torch.zeros(n_single * nkv, dtype=torch.int32, device=qkv.device))
        if mfma and nsplit > planned and n_single <= DECODE_LIST_MAX_TOKENS:
            # contexts that differ: one run length for the batch and the list of the runs that have keys, made
            # on the device from the context lengths, once a step for all layers with these numbers (a
            # recorded step makes them again at every replay)
            key = ("decode_run_keys", nkv, int(window), nsplit, meta.max_blocks, n_single)
            run_keys = meta.extra.get(key)
            if run_keys is None:
                # one buffer for every number of runs and (growing only with the batch) of tokens: a
                # name per combination would pile up over a serving run
                name = "attn.run_keys.%d.%d.%d" % (getattr(meta, "group", 0), nkv, int(window))
                size = 2 + n_single + n_single * DECODE_MAX_SPLITS
                run_keys = (ws.buffer(name, (size,), torch.int32) if ws is not None
                            else torch.empty(size, dtype=torch.int32, device=qkv.device))
                decode_run_keys(meta, lst, n_single, page_size, window, nkv, nsplit, _simd_count(qkv.device), run_keys,
                                group=quad)
                meta.extra[key] = run_keys
        _run("attention", "li_paged_attention_decode", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), _DT[qkv.dtype], bt.data_ptr(), meta.max_blocks,
             0 if lst is None else lst.data_ptr(), n_single, meta.seg_of_token.data_ptr(),
             meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             0 if acc is None else acc.data_ptr(), 0 if ml is None else ml.data_ptr(),
             nh, nkv, dh, page_size, k.shape[0], int(window), float(scale), nsplit,
             (2 if quad == 1 and nsplit > 1 else 1) if mfma else 0,
             0 if run_keys is None else run_keys.data_ptr(), 0 if done is None else done.data_ptr())
    # the matrix-core kernel for portions keeps a tile's pages in LDS (8192 entries) and divides
    # positions by the page size in float, exact below 2^21 keys; longer tables take the general kernel
    if (n_multi and qkv.dtype is torch.bfloat16 and dh in (64, 128) and meta.num_tiles
            and meta.tile_rows == PREFILL_TILE_ROWS and n_multi == meta.num_multi and meta.max_blocks <= 8192 and meta.max_blocks * page_size <= 1 << 21):
        # few tiles against long contexts: the tiles' keys in runs, joined by the kernel that joins the
        # decode attention's (the library says how many; their results take room in the workspace)
        runs = 1
        if ws is not None:
            runs = _prefill_runs(getattr(meta, "host_q_len", None), getattr(meta, "host_ctx_len", None), nh, nkv, dh,
                                 meta.max_blocks, window, t)
        acc = ml = lst = None
        if runs > 1:
            acc = ws.buffer("attn.runs_acc", (t, nh, runs, dh), torch.float32)
            ml = ws.buffer("attn.runs_ml", (t, nh, runs, 2), torch.float32)
            lst = meta.multi_tokens if n_multi < t else None
        _run("attention", "li_paged_attention_prefill", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), bt.data_ptr(), meta.max_blocks, meta.tiles.data_ptr(),
             meta.num_tiles, meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             nh, nkv, dh, page_size, k.shape[0], int(window), float(scale), runs,
             0 if acc is None else acc.data_ptr(), 0 if ml is None else ml.data_ptr(),
             0 if lst is None else lst.data_ptr(), n_multi)
    elif (n_multi and qkv.dtype is torch.float32 and dh in (64, 128) and meta.num_tiles
            and meta.tile_rows == PREFILL_TILE_ROWS and n_multi == meta.num_multi):
        # the 32-bit path's tiled kernel for portions (other head sizes: the general kernel below)
        _run("attention", "li_paged_attention_prefill_f32", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), bt.data_ptr(), meta.max_blocks, meta.tiles.data_ptr(),
             meta.num_tiles, meta.q_start.data_ptr(), meta.q_len.data_ptr(), meta.ctx_len.data_ptr(),
             nh, nkv, dh, page_size, k.shape[0], int(window), float(scale))
    elif n_multi:
        lst = meta.multi_tokens if n_multi < t else None
        _run("attention", "li_paged_attention", qkv.data_ptr(), qkv.stride(0), out.data_ptr(),
             k.data_ptr(), v.data_ptr(), _DT[qkv.dtype], bt.data_ptr(), meta.max_blocks,
             0 if lst is None else lst.data_ptr(), meta.seg_of_token.data_ptr(), meta.q_start.data_ptr(),
             meta.q_len.data_ptr(), meta.ctx_len.data_ptr(), meta.num_segments, n_multi, meta.max_q_len,
             meta.max_ctx_len, nh, nkv, dh, page_size, k.shape[0], int(window), float(scale))


# ------------------------------------------------------------------ sampling
_argmax_scratch = {}
_sample_scratch = {}


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[i] = index of the maximum of row i, the lowest index on ties."""
    _gpu(logits, out)
    _chk(logits.dim() == 2 and logits.dtype is torch.float32 and logits.is_contiguous(), "argmax: logits")
    _chk(out.dtype is torch.int32 and out.numel() == logits.shape[0] and out.is_contiguous(), "argmax: out")
    n = logits.shape[0]
    if n:
        key = (logits.device, n)
        if key not in _argmax_scratch:
            _argmax_scratch[key] = (torch.empty(n * 32, dtype=torch.float32, device=logits.device),
                                    torch.empty(n * 32, dtype=torch.int32, device=logits.device))
        sv, si = _argmax_scratch[key]
        _run("sampling", "li_argmax_rows", logits.data_ptr(), out.data_ptr(), sv.data_ptr(), si.data_ptr(),
             n, logits.shape[1])


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
                top_p: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor) -> None:
    """One token per row.  temperature <= 0: the argmax (lowest index on ties).
    Otherwise the candidates, ordered by (logit descending, index ascending),
    are cut to the first top_k (when 0 < top_k < V) and then to the shortest
    prefix whose softmax mass among them reaches top_p (when 0 < top_p < 1);
    the softmax of logits/temperature over the survivors is sampled by inverse
    CDF over ascending ids with the row's uniform number in [0, 1)."""
    _gpu(logits, temperature, top_k, top_p, uniform, out)
    _chk(logits.dim() == 2 and logits.dtype is torch.float32 and logits.is_contiguous(), "sample: logits")
    n = logits.shape[0]
    for t_, dt in ((temperature, torch.float32), (top_k, torch.int32), (top_p, torch.float32),
                   (uniform, torch.float32), (out, torch.int32)):
        _chk(t_.dtype is dt and t_.numel() == n and t_.is_contiguous(), "sample: per-row arrays")
    if n:
        v = logits.shape[1]
        key = (logits.device, n, v)
        if key not in _sample_scratch:               # what the first of the two kernels leaves for the second
            _sample_scratch[key] = torch.empty(_sample_scratch_floats(n, v), dtype=torch.float32, device=logits.device)
        tiles = _sample_scratch[key]
        _run("sampling", "li_sample_rows", logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(),
             top_p.data_ptr(), uniform.data_ptr(), out.data_ptr(), n, v, tiles.data_ptr(), tiles.numel())


SAMPLE_SLOT_WORDS = 8          # 32-bit words of a slot's row in the sampling table (csrc/sampling.hip)
SAMPLE_ROW_GREEDY = 1 << 24    # flag of a step's row: greedy whatever its slot's row says


def sample_prepare(rows: torch.Tensor, table: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
                   top_p: torch.Tensor, uniform: torch.Tensor) -> None:
    """From the sampling table of the state slots (int32 [slots, 8]: temperature and top_p as float bits,
    top_k, the seed's two halves, the draws so far) and a step's rows (int32: slot | flags << 24), the
    per-row arrays that `sample_rows` takes; the uniform number of every sampling row is drawn on the
    device from its slot's seed and count, and the count goes up."""
    _gpu(rows, table, temperature, top_k, top_p, uniform)
    n = rows.numel()
    _chk(rows.dtype is torch.int32 and rows.is_contiguous(), "sample_prepare: rows must be int32")
    _chk(table.dtype is torch.int32 and table.dim() == 2 and table.shape[1] == SAMPLE_SLOT_WORDS and table.is_contiguous(),
         "sample_prepare: the table must be int32 [slots, 8]")
    for t_, dt in ((temperature, torch.float32), (top_k, torch.int32), (top_p, torch.float32), (uniform, torch.float32)):
        _chk(t_.dtype is dt and t_.numel() == n and t_.is_contiguous(), "sample_prepare: per-row arrays")
    if n:
        _run("sampling", "li_sample_prepare", rows.data_ptr(), n, table.data_ptr(), table.shape[0],
             temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), uniform.data_ptr())
