"""Specifications that describe a model as data.

A model is a list of layers, each a block arrangement that names its parts
(norms, a mixer, a feed-forward), and an execution order over those layers.
Every part is given by a `PartSpec`: the registry key of its class, the prefix
of its tensors in the checkpoint, and its sizes and constants.  Nothing here
knows a particular architecture; an architecture is a function from its typed
configuration to a `ModelSpec`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: `kind` is looked up in the parts registry under the category
    the holder expects (norm, mixer, feed_forward, position, block, embedding,
    head); `prefix` is prepended to the part's own tensor names; `args` holds
    its sizes and constants."""
    kind: str
    prefix: str = ""
    args: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """A layer: the arrangement (`block`) and the parts it arranges, by role.
    The pre-norm arrangement has the roles norm1, mixer, norm2, feed_forward."""
    block: str
    parts: Dict[str, PartSpec]


@dataclass(frozen=True)
class ExecEntry:
    """One entry of the execution order: run layer `layer`; if `cache_from` is
    given, the mixer writes nothing and reads the cache that entry
    `cache_from` of the order (an earlier one) wrote."""
    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[ExecEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("model spec: no layers")
        if not self.order:
            raise ValueError("model spec: empty execution order")
        for i, e in enumerate(self.order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"model spec: order[{i}] names layer {e.layer}, "
                                 f"there are {len(self.layers)}")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ValueError(f"model spec: order[{i}] reads the cache of entry "
                                     f"{e.cache_from}, which is not an earlier entry")
                if self.order[e.cache_from].cache_from is not None:
                    raise ValueError(f"model spec: order[{i}] reads the cache of entry "
                                     f"{e.cache_from}, which owns no cache itself")
