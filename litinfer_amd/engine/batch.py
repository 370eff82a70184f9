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

from ..cache import native
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
    # What follows is laid out only when a part of the model asks for it (`Part.batch_needs`).
    # tokens of segments that bring ONE token (decoding) and the other tokens, as lists of token
    # numbers; None when all tokens of the batch are of that kind (then no list is needed)
    single_tokens: Optional[torch.Tensor] = None
    num_single: int = 0
    multi_tokens: Optional[torch.Tensor] = None
    num_multi: int = 0
    # the tokens of segments with several tokens, cut into tiles of up to `tile_rows` consecutive
    # tokens of one segment: int32 [tiles, 4] = (segment, first token, tokens, 0)
    tiles: Optional[torch.Tensor] = None
    num_tiles: int = 0
    tile_rows: int = 0
    max_single_ctx: int = 0
    group: int = 0                   # the page group whose tables these are
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
        for meta in self._attn:
            meta.extra.clear()

    def shared(self, key, make: Callable[[], Any]):
        """Per-step value shared by every part that asks with the same key."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]


def build_context(cache, entries: Sequence[StepEntry], ws, uploader: "BatchUploader",
                  pad_blocks: Optional[Sequence[int]] = None, feedback: Optional[torch.Tensor] = None,
                  needs=None, handles=None) -> StepContext:
    """Lay out the step's integers (see the module text) for the given entries
    against the cache's current tables, upload them, and return the context.
    Pages for the entries' tokens must have been reserved.  `pad_blocks` gives,
    per page group, a width to pad the block tables to (for steps that are
    replayed from a recorded graph, whose array shapes must not change).
    `needs` (a `parts.BatchNeeds`) says which further index arrays the model's parts
    want: tiles of some number of tokens, the lists of single and multi tokens.
    The arrays are filled by the host library straight into the pinned buffer
    (csrc/host.cpp, li_book_build_batch)."""
    lib = native.lib()
    ng = len(cache.groups)
    nseg = len(entries)
    if handles is None:
        handles = np.fromiter((cache.handle(e.rid) for e in entries), dtype=np.int64, count=nseg)
    q_len = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=nseg)
    if int(q_len.max()) == 1:                        # single tokens all: no array per entry
        ids = np.fromiter((e.tokens[0] for e in entries), dtype=np.int32, count=nseg)
    else:
        ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
    id_src = None
    if any(e.take is not None for e in entries):
        if feedback is None:
            raise ValueError("step: an entry takes tokens from the feedback buffer, but there is none")
        if int(q_len.max()) == 1:
            id_src = np.fromiter((-1 if e.take is None else e.take[0] for e in entries), dtype=np.int32, count=nseg)
        else:
            id_src = np.concatenate([np.full(len(e.tokens), -1, dtype=np.int32) if e.take is None
                                     else np.asarray(e.take, dtype=np.int32) for e in entries])
    want_off = np.zeros(nseg + 1, dtype=np.int32)
    np.cumsum([len(e.want) for e in entries], out=want_off[1:])
    want = np.fromiter((int(w) for e in entries for w in e.want), dtype=np.int32, count=int(want_off[-1]))
    pad = None if pad_blocks is None else np.asarray(pad_blocks, dtype=np.int32)
    tile_rows = int(needs.tile_rows) if needs is not None else 0
    token_kinds = bool(needs.token_kinds) if needs is not None else False
    offsets = np.zeros(12 + 2 * ng, dtype=np.int64)
    info = np.zeros(8 + max(ng, 1), dtype=np.int32)

    def ptr(a):
        return None if a is None else a.ctypes.data

    def call(out_ptr, cap):
        n = lib.li_book_build_batch(cache.book, nseg, ptr(handles), ptr(q_len), ptr(ids), ptr(id_src),
                                    ptr(want_off), ptr(want), ptr(pad), tile_rows, int(token_kinds), out_ptr, cap,
                                    ptr(offsets), ptr(info))
        if n < 0:
            raise AssertionError(cache._error())
        return int(n)
    total = call(None, 0)
    host = uploader.stage(total)
    call(host.data_ptr(), host.numel())
    dev = uploader.push(total)
    T, nwant, nsingle, nmulti, ntiles, max_q, max_ctx, max_single_ctx = (int(x) for x in info[:8])
    hv = host.numpy()

    def d(k, n, shape=None):
        t = dev[int(offsets[k]):int(offsets[k]) + n]
        return t if shape is None else t.view(shape)

    def h(k, n):
        return hv[int(offsets[k]):int(offsets[k]) + n].copy()
    ctx = StepContext(ws, T, nseg)
    ctx.ids, ctx.positions = d(0, T), d(1, T)
    d_seg, d_qs, d_ql, d_cl = d(2, T), d(3, nseg), d(4, nseg), d(5, nseg)
    ctx.state_slots, ctx.want_rows = d(6, nseg), d(7, nwant)
    d_single = d(8, nsingle) if token_kinds else None
    d_multi = d(9, nmulti) if token_kinds else None
    d_tiles = d(10, ntiles * 4, (ntiles, 4)) if tile_rows else None
    ctx.id_src = d(11, T) if feedback is not None else None
    ctx.feedback = feedback
    ctx.num_want = nwant
    ctx.host_state_slots = h(6, nseg)
    ctx.host_q_start, ctx.host_q_len, ctx.host_ctx_len = h(3, nseg), h(4, nseg), h(5, nseg)
    P = cache.page_size
    for gi in range(ng):
        mb = int(info[8 + gi])
        ctx._slot_maps.append(d(13 + 2 * gi, T))
        ctx._attn.append(AttentionMeta(
            block_table=d(12 + 2 * gi, nseg * mb, (nseg, mb)), max_blocks=mb, seg_of_token=d_seg, q_start=d_qs,
            q_len=d_ql, ctx_len=d_cl, num_segments=nseg, num_tokens=T,
            max_q_len=max_q, max_ctx_len=max_ctx,
            host_q_start=ctx.host_q_start, host_q_len=ctx.host_q_len, host_ctx_len=ctx.host_ctx_len,
            single_tokens=d_single if nmulti else None, num_single=nsingle,
            multi_tokens=d_multi if nsingle else None, num_multi=nmulti,
            tiles=d_tiles, num_tiles=ntiles, tile_rows=tile_rows, group=gi,
            # with padded tables the split count must not follow the context either
            max_single_ctx=(mb * P if pad_blocks is not None else max_single_ctx)))
    return ctx
