"""The batch of one step: ragged segments of (request, its next tokens).

All integer metadata of a step is laid out in one host array and reaches the
device in one copy: token ids, positions, the segment of each token, per
segment the offset of its first token, its length, the context length after
the step and its state slot, the rows whose logits are wanted, and per page
group the block tables [segments, max_blocks] and the page slot of every
token.  The reference builds the same flat layout (src/llaisys/models/qwen2.cpp:942-957)
but uploads the tables again for every layer (:993-1007).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..utils.pinned import BatchUploader


@dataclass
class StepEntry:
    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()          # places among `tokens` whose logits are asked for
    # For each of `tokens`, -1 or a place in the engine's feedback buffer (`Engine.feedback`): the
    # token's id is then read from there when the step runs, and the number in `tokens` is not
    # used.  This is how a token sampled on the device enters the next step before the host knows it.
    take: Optional[Sequence[int]] = None


@dataclass
class AttentionMeta:
    """Device arrays the attention kernels index, and the host numbers their
    launches are sized by."""
    block_table: torch.Tensor        # [segments, max_blocks] int32, -1 = given back
    max_blocks: int
    seg_of_token: torch.Tensor       # [T]
    q_start: torch.Tensor            # [segments]
    q_len: torch.Tensor              # [segments]
    ctx_len: torch.Tensor            # [segments]  cached length after this step
    num_segments: int
    num_tokens: int
    max_q_len: int
    max_ctx_len: int
    host_q_start: np.ndarray
    host_q_len: np.ndarray
    host_ctx_len: np.ndarray
    # tokens of segments that bring ONE token (decoding) and the other tokens, as lists of token
    # numbers; None when all tokens of the batch are of that kind (then no list is needed)
    single_tokens: Optional[torch.Tensor] = None
    num_single: int = 0
    multi_tokens: Optional[torch.Tensor] = None
    num_multi: int = 0
    # the tokens of segments with several tokens, cut into tiles of up to 32 consecutive tokens
    # of one segment: int32 [tiles, 4] = (segment, first token, tokens, 0)
    tiles: Optional[torch.Tensor] = None
    num_tiles: int = 0
    max_single_ctx: int = 0
    extra: Dict[Any, Any] = field(default_factory=dict)    # what kernels derive and keep for the step


class StepContext:
    """What parts may read during a step."""

    def __init__(self, ws, num_tokens: int, num_segments: int):
        self.ws = ws
        self.num_tokens = num_tokens
        self.num_segments = num_segments
        self.ids: torch.Tensor = None
        self.id_src: torch.Tensor = None              # [T] int32: place in `feedback` or -1
        self.feedback: torch.Tensor = None            # the engine's buffer of ids chosen on the device
        self.positions: torch.Tensor = None
        self.state_slots: torch.Tensor = None        # [segments] int32, device
        self.host_state_slots: np.ndarray = None
        self.host_q_start: np.ndarray = None
        self.host_q_len: np.ndarray = None
        self.host_ctx_len: np.ndarray = None
        self.want_rows: torch.Tensor = None
        self.num_want = 0
        self._slot_maps: List[torch.Tensor] = []
        self._attn: List[AttentionMeta] = []
        self._shared: Dict[Any, Any] = {}

    def slot_map(self, group: int) -> torch.Tensor:
        return self._slot_maps[group]

    def attention_meta(self, group: int) -> AttentionMeta:
        return self._attn[group]

    def forget_shared(self) -> None:
        self._shared.clear()

    def shared(self, key, make: Callable[[], Any]):
        """Per-step value shared by every part that asks with the same key."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]


def build_context(cache, entries: Sequence[StepEntry], ws, uploader: "BatchUploader",
                  pad_blocks: Optional[Sequence[int]] = None, feedback: Optional[torch.Tensor] = None) -> StepContext:
    """Lay out the step's integers (see the module text) for the given entries
    against the cache's current tables, upload them, and return the context.
    Pages for the entries' tokens must have been reserved.  `pad_blocks` gives,
    per page group, a width to pad the block tables to (for steps that are
    replayed from a recorded graph, whose array shapes must not change)."""
    P = cache.page_size
    nseg = len(entries)
    q_len = np.array([len(e.tokens) for e in entries], dtype=np.int32)
    q_start = np.zeros(nseg + 1, dtype=np.int32)
    np.cumsum(q_len, out=q_start[1:])
    T = int(q_start[-1])
    cached = np.array([cache.cached_len(e.rid) for e in entries], dtype=np.int32)
    ctx_len = cached + q_len
    ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
    id_src = np.full(T, -1, dtype=np.int32)
    for i, e in enumerate(entries):
        if e.take is not None:
            id_src[q_start[i]:q_start[i + 1]] = np.asarray(e.take, dtype=np.int32)
    seg_of_token = np.repeat(np.arange(nseg, dtype=np.int32), q_len)
    pos = (np.arange(T, dtype=np.int32) - q_start[seg_of_token] + cached[seg_of_token]).astype(np.int32)
    slots = np.array([cache.slot(e.rid) for e in entries], dtype=np.int32)
    want = [int(q_start[i]) + int(w) for i, e in enumerate(entries) for w in e.want]
    want_rows = np.asarray(want, dtype=np.int32)
    single_mask = q_len[seg_of_token] == 1
    single = np.nonzero(single_mask)[0].astype(np.int32)
    multi = np.nonzero(~single_mask)[0].astype(np.int32)
    tile_rows = [(i, int(q_start[i]) + a, min(32, int(q_len[i]) - a), 0)
                 for i in range(nseg) if q_len[i] > 1 for a in range(0, int(q_len[i]), 32)]
    tiles = np.asarray(tile_rows, dtype=np.int32).reshape(-1, 4)
    parts = [ids, pos, seg_of_token, q_start[:-1].copy(), q_len, ctx_len, slots, want_rows, single, multi, tiles,
             id_src]
    tables, max_blocks = [], []
    for gi in range(len(cache.groups)):
        tabs = [cache.block_table(e.rid, gi) for e in entries]
        mb = max(1, max(len(t) for t in tabs))
        if pad_blocks is not None:
            mb = max(mb, int(pad_blocks[gi]))
        tab = np.full((nseg, mb), -1, dtype=np.int32)
        for i, t in enumerate(tabs):
            tab[i, :len(t)] = t
        page = tab[seg_of_token, pos // P]
        if (page < 0).any():
            raise AssertionError("step: a token of the batch has no page")
        slot_map = (page.astype(np.int64) * P + pos % P).astype(np.int32)
        tables.append(tab)
        max_blocks.append(mb)
        parts += [tab, slot_map]
    dev = uploader.upload(parts)
    ctx = StepContext(ws, T, nseg)
    (ctx.ids, ctx.positions, d_seg, d_qs, d_ql, d_cl, ctx.state_slots, ctx.want_rows,
     d_single, d_multi, d_tiles, ctx.id_src) = dev[:12]
    ctx.feedback = feedback
    if feedback is None:
        if (id_src >= 0).any():
            raise ValueError("step: an entry takes tokens from the feedback buffer, but there is none")
        ctx.id_src = None
    ctx.num_want = len(want)
    ctx.host_state_slots = slots
    ctx.host_q_start, ctx.host_q_len, ctx.host_ctx_len = q_start[:-1], q_len, ctx_len
    for gi in range(len(cache.groups)):
        d_tab, d_slot = dev[12 + 2 * gi], dev[13 + 2 * gi]
        ctx._slot_maps.append(d_slot)
        ctx._attn.append(AttentionMeta(
            block_table=d_tab, max_blocks=max_blocks[gi], seg_of_token=d_seg, q_start=d_qs,
            q_len=d_ql, ctx_len=d_cl, num_segments=nseg, num_tokens=T,
            max_q_len=int(q_len.max()), max_ctx_len=int(ctx_len.max()),
            host_q_start=q_start[:-1], host_q_len=q_len, host_ctx_len=ctx_len,
            single_tokens=d_single if len(multi) else None, num_single=len(single),
            multi_tokens=d_multi if len(single) else None, num_multi=len(multi),
            tiles=d_tiles, num_tiles=len(tile_rows),
            # with padded tables the split count must not follow the context either
            max_single_ctx=(max_blocks[gi] * P if pad_blocks is not None else
                            int(ctx_len[q_len == 1].max()) if len(single) else 0)))
    return ctx
