"""Interfaces of the parts a layer is put together from, and their registry.

A part is built from a `PartSpec` (its sizes and constants, and the prefix of
its tensors) and a `Runtime` (device and activation dtype).  It says which
tensors it expects, takes them, and then runs on the step's batch.  No part
knows which model it is in; the model and the block only use what is written
here.

Interfaces (T = tokens of the step, H = hidden size):

* Norm.forward(x [T, H] float32, out) -> out [T, H] in the activation dtype.
* Mixer.cache_need() -> PagedNeed (named tensors per token, in pages; PagedKVNeed(...)
  builds the usual keys and values) | StateNeed | None, or a tuple of them (pages AND
  state of fixed size: one paged need and any number of named state needs);
  Mixer.forward(xn [T, H], residual, ctx, cache): ADDS its output to the
  residual stream in 32-bit.  `residual` is a `ResidualStream`
  (parts/stream.py): `residual.add_linear(linear, h)` adds h W^T + b, and
  `residual.tensor()` is the float32 tensor [T, H] itself for a part that adds
  in its own way.  `cache` is the CacheView of the entry of the execution order
  that is running; `cache.owned` is False when the entry reads another entry's
  cache and must write nothing.
* FeedForward.forward(xn, residual, ctx): adds its output to the stream.
* Position: prepares per-step tables and rotates (or otherwise encodes) the
  mixer's queries and keys; see `parts/position.py`.
* Block.forward(stream, ctx, cache): runs its parts on the `ResidualStream`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ..config.spec import PartSpec
from ..weights.loader import ParamSpec


@dataclass(frozen=True)
class Runtime:
    """Where and in which precision a model runs.  `dtype` is the activation and
    matrix dtype: torch.bfloat16 (serving) or torch.float32 (everything in true
    32-bit).  One dtype holds for every matrix of the model, whatever the checkpoint
    stores them in, as the reference decides one dtype for the whole model and
    converts every tensor to it (python/llaisys/models/qwen2.py:88-110, 253-264).
    `keep_stored_precision` (off by default) leaves a matrix that is stored in 32-bit
    (or in half precision, which is widened) in 32-bit inside the bfloat16 engine;
    its products then run in the 32-bit kernels, slower and on twice the bytes."""
    device: torch.device
    dtype: torch.dtype
    keep_stored_precision: bool = False
    # stored dtype -> number of matrices that were rounded to bfloat16 when they were bound
    rounded: Dict[str, int] = field(default_factory=dict, compare=False, hash=False)

    def matrix(self, t: torch.Tensor) -> torch.Tensor:
        """A stored matrix as this runtime multiplies with it.  In 32-bit mode
        everything is widened (exactly).  In bfloat16 mode a matrix stored in
        another precision is rounded once, to nearest even, to bfloat16, so that
        every product takes the bfloat16 kernels (unless `keep_stored_precision`)."""
        if self.dtype is torch.float32:
            t = t.to(torch.float32)
        elif t.dtype is not torch.bfloat16 and t.is_floating_point() and not self.keep_stored_precision:
            self.rounded[str(t.dtype)] = self.rounded.get(str(t.dtype), 0) + 1
            t = t.to(self.device).to(torch.bfloat16)      # (rounded on the device: a large table takes a moment on the host)
        return t.to(self.device).contiguous()

    def vector(self, t: torch.Tensor) -> torch.Tensor:
        """Norm weights and biases are held in float32 in both modes."""
        return t.to(torch.float32).to(self.device).contiguous()


@dataclass(frozen=True)
class PagedTensor:
    """One tensor that a mixer keeps for every token of a request, in pages: `shape` is
    what one token holds, e.g. (kv_heads, head_dim) for keys or (latent,) for a compressed
    cache; `dtype` None means the engine's activation dtype.  A page of it is laid out as
    [*shape[:-1], page_size, shape[-1]]: the rows of one head lie together."""
    name: str
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        return (*self.shape[:-1], page_size, self.shape[-1])


@dataclass(frozen=True)
class PagedNeed:
    """What a mixer keeps per token in pages: any number of named tensors of any shapes;
    `window` > 0 keeps only the last `window` positions visible (older pages are given
    back).  Entries of the execution order with equal needs share a page group: one page
    id and one block table per request serve all of them."""
    tensors: Tuple[PagedTensor, ...]
    window: int = 0

    def bytes_per_token(self, default_dtype: torch.dtype) -> int:
        total = 0
        for t in self.tensors:
            n = 1
            for s in t.shape:
                n *= int(s)
            total += n * torch.empty((), dtype=t.dtype or default_dtype).element_size()
        return total


def PagedKVNeed(num_kv_heads: int, head_dim: int, window: int = 0) -> PagedNeed:
    """Keys and values of equal shape (kv_heads, head_dim), named "k" and "v": what the
    attention of the reference keeps (src/llaisys/kv_cache/block_kv_cache.hpp:16-63)."""
    shape = (int(num_kv_heads), int(head_dim))
    return PagedNeed((PagedTensor("k", shape), PagedTensor("v", shape)), int(window))


@dataclass(frozen=True)
class BatchNeeds:
    """Index arrays, beyond the basic ones, that a part's kernels want laid out with a
    step's batch (they travel in the step's one upload).  `tile_rows` > 0: the tokens of
    segments with several tokens cut into tiles of up to that many consecutive tokens of one
    segment; `token_kinds`: the lists of tokens of single-token segments and of the others.
    `row_tile` is no array but a hint for whoever cuts prompts into steps: the part's kernels take
    a step's rows that many at a time, so a step of a few rows more than a multiple of it costs a
    whole tile more (1: no such tile).  The model's is the largest of its parts'."""
    tile_rows: int = 0
    token_kinds: bool = False
    row_tile: int = 1

    def merged(self, other: "BatchNeeds") -> "BatchNeeds":
        if self.tile_rows and other.tile_rows and self.tile_rows != other.tile_rows:
            raise ValueError(f"parts ask for tiles of {self.tile_rows} and of {other.tile_rows} tokens; "
                             f"a step's batch is laid out with one tile size")
        return BatchNeeds(self.tile_rows or other.tile_rows, self.token_kinds or other.token_kinds,
                          max(self.row_tile, other.row_tile))


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size, zero when a request is admitted.  A mixer that keeps
    several gives them different names."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    name: str = "state"


def needs_of(need) -> Tuple[Optional[PagedNeed], Tuple[StateNeed, ...]]:
    """What `cache_need()` returned (None, one need, or a tuple or list of needs), taken apart:
    the paged need (at most one per entry of the execution order; its tensors are any number) and
    the state needs (any number, with distinct names)."""
    items = () if need is None else tuple(need) if isinstance(need, (tuple, list)) else (need,)
    paged = [n for n in items if isinstance(n, PagedNeed)]
    states = tuple(n for n in items if isinstance(n, StateNeed))
    if len(paged) + len(states) != len(items):
        bad = [n for n in items if not isinstance(n, (PagedNeed, StateNeed))]
        raise TypeError(f"cache need {bad[0]!r} is neither a PagedNeed nor a StateNeed")
    if len(paged) > 1:
        raise ValueError("a mixer keeps ONE paged need (of any number of tensors); two page groups for one entry "
                         "of the execution order are not supported")
    if len({s.name for s in states}) != len(states):
        raise ValueError(f"state needs of one mixer need distinct names, found {[s.name for s in states]}")
    return (paged[0] if paged else None), states


class Part:
    category = "part"
    # True if `forward` only launches work whose arguments are device arrays and sizes of the batch
    # (tokens, segments, table width): then a decode step may be recorded once as a HIP graph and
    # replayed.  A part that reads the step's host-side arrays must leave this False.
    graph_safe = False

    def __init__(self, spec: PartSpec, rt: Runtime):
        self.spec = spec
        self.rt = rt
        self.prefix = spec.prefix

    def expected_params(self) -> Dict[str, ParamSpec]:
        """Full tensor name -> ParamSpec."""
        return {}

    def batch_needs(self) -> BatchNeeds:
        """What this part's kernels want laid out with a step's batch beyond ids, positions,
        segments, block tables and page slots (nothing, for most parts)."""
        return BatchNeeds()

    def load_params(self, get: Callable[[str], Optional[torch.Tensor]]) -> None:
        """`get(name)` returns the stored tensor on the CPU, or None when an
        optional tensor is absent."""


@dataclass(frozen=True)
class RmsScaling:
    """An RMS norm, y = weight * x / sqrt(mean(x^2) + eps), in the form in which the
    products on its two sides can take it over: the one before writes weight * x, the
    one after scales its rows by 1 / sqrt(mean(x^2) + eps)."""
    weight: torch.Tensor          # float32 [size]
    eps: float


@dataclass
class ScaledRows:
    """The input of a norm as the product before it left it: `rows` = weight * x
    in the engine's dtype, `scale` what the product after it needs for the rows'
    factors (an `ops.RowScale`)."""
    rows: torch.Tensor
    scale: Any


class Norm(Part):
    category = "norm"

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def as_scaling(self) -> Optional[RmsScaling]:
        """How the products on the two sides of this norm can share it between them
        (an RmsScaling), or None: then the norm is always a pass of its own."""
        return None


class Mixer(Part):
    category = "mixer"

    def cache_need(self):
        return None

    def forward(self, xn, residual, ctx, cache) -> None:
        raise NotImplementedError

    def forward_prenorm(self, norm: Norm, residual, xn, ctx, cache) -> None:
        """x += mixer(norm(x)) for the residual stream x; `xn` is room for the
        normed rows.  The default norms in a pass of its own.  A mixer whose first
        product can scale its rows overrides this and asks the stream for
        `scaled_rows(norm)`, which the product before the norm may have left."""
        self.forward(residual.normed(norm, xn), residual, ctx, cache)


class FeedForward(Part):
    category = "feed_forward"

    def forward(self, xn, residual, ctx) -> None:
        raise NotImplementedError

    def forward_prenorm(self, norm: Norm, residual, xn, ctx) -> None:
        """x += feed_forward(norm(x)); see Mixer.forward_prenorm."""
        self.forward(residual.normed(norm, xn), residual, ctx)


class Block(Part):
    category = "block"

    def cache_need(self):
        return None

    def first_norm(self) -> Optional[Norm]:
        """The norm through which this block first reads the residual stream, if
        that is how it begins: the block before it is told, so that its last
        product can prepare the rows."""
        return None

    def forward(self, x, ctx, cache) -> None:
        raise NotImplementedError


_PARTS: Dict[Tuple[str, str], type] = {}


def register_part(category: str, kind: str, cls: type) -> None:
    _PARTS[(category, kind)] = cls


def build_part(category: str, spec: PartSpec, rt: Runtime, **extra) -> Any:
    key = (category, spec.kind)
    if key not in _PARTS:
        known = sorted(k for c, k in _PARTS if c == category)
        raise KeyError(f"no {category} part named '{spec.kind}'; registered: {', '.join(known)}")
    return _PARTS[key](spec, rt, **extra)
