"""The engine: a model, its cache and ONE step function.

`step(entries)` takes a batch of (request, its next tokens): portions of
prompts beside single decoded tokens, cut anywhere.  It runs only the tokens
it is given, as one batch, against the cache that earlier steps left, and
returns float32 logits at the wanted places.  Generation (the scheduler) and
trace replay are two callers of this one function.

The reference's step builds its batch itself from its request list and admits
only whole prompts and single tokens (src/llaisys/models/qwen2.cpp:922-957);
its attention already derives each query's horizon as ctx - qlen + i
(src/ops/paged_attention/op.cpp:204), which is what makes portions sound.
"""
from __future__ import annotations

import os
import sys
from collections import OrderedDict
from pathlib import Path
from typing import Any, Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheFull, CacheManager, group_needs
from ..config import load_config, lookup, architecture_name
from ..config.spec import ModelSpec
from ..parts.base import Runtime
from ..utils.profiler import profiler, trace_enabled
from ..weights import load_into, random_tensor
from .batch import BatchUploader, StepContext, StepEntry, build_context
from .model import Model
from .workspace import Workspace

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
          "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"engine dtype must be bfloat16 or float32, found {dtype}")
        return dtype
    if str(dtype) not in DTYPES:
        raise ValueError(f"engine dtype must be one of {sorted(DTYPES)}, found {dtype!r}")
    return DTYPES[str(dtype)]


FEEDBACK_SLOTS = 4096


class StepError(ValueError):
    """The batch is not valid; nothing was changed."""


class Engine:
    def __init__(self, spec: ModelSpec, *, dtype="bfloat16", device="cuda:0", page_size: int = 16,
                 num_pages: Optional[int] = None, max_tokens: Optional[int] = None,
                 max_seqs: int = 64, page_order_seed: Optional[int] = None,
                 config: Any = None, use_graphs: bool = True, graph_after: int = 2,
                 keep_stored_precision: bool = False, max_graphs: int = 64, step_tokens: int = 2048,
                 pad_rows_to: int = 4):
        """keep_stored_precision: with dtype bfloat16, leave matrices that the checkpoint stores in
        32-bit or half precision in 32-bit (their products then run in the 32-bit kernels) instead of
        rounding them once to bfloat16 when they are bound."""
        self.spec = spec
        self.config = config
        self.rt = Runtime(torch.device(device), parse_dtype(dtype), bool(keep_stored_precision))
        if self.rt.device.type == "cuda":
            from ..kernels import ops
            ops.require_gpu(self.rt.device)
        self.model = Model(spec, self.rt)
        self.page_size = int(page_size)
        self.max_seqs = int(max_seqs)
        self._num_pages = num_pages
        # the most tokens a step is expected to bring: sizes the pools of windowed groups (see _make_cache)
        self.step_tokens = max(1, int(step_tokens))
        self._max_tokens = max_tokens
        self._page_order_seed = page_order_seed
        self.cache: Optional[CacheManager] = None
        self.ws = Workspace(self.rt.device)
        self._uploader = BatchUploader(self.rt.device)
        # ids of tokens chosen on the device (a sampler's output): an entry of the NEXT step may
        # take its token from here (`StepEntry.take`), so the host need not wait for the number
        self.feedback = torch.zeros(FEEDBACK_SLOTS, dtype=torch.int32, device=self.rt.device)
        self.steps_run = 0
        self.unused_weights: List[str] = []
        # decode steps (every request brings one token) are recorded as HIP graphs, one per batch
        # shape, and replayed: a step is some hundred small launches otherwise
        self.use_graphs = bool(use_graphs) and self.rt.device.type == "cuda" and not profiler.enabled
        # A decode step of a shape (requests, wanted rows, table widths) is recorded at its graph_after-th
        # occurrence and replayed from then on; before that it runs eagerly (the first occurrence sizes the
        # buffers).  The recording runs in the eager pass's place, on a stream of its own and without a
        # device-wide wait (`_record`), so that a recorded step costs what an eager one costs: where requests
        # come and go a shape lasts a few steps only, and a recording that cost several steps' time (as one
        # made with `torch.cuda.graph` after the eager pass did) ate what the replays gave back.
        self.graph_after = max(2, int(graph_after))
        self._trace = trace_enabled()
        # shape -> ("seen", times) | ("graph", graph, its output), least recently used first; at most
        # `max_graphs` recorded ones are kept
        self._graphs: "OrderedDict[Any, Any]" = OrderedDict()
        self.max_graphs = max(1, int(max_graphs))
        # recorded steps of more than `pad_rows_to` requests take whole multiples of it (see `step`); 1: as they come
        self.pad_rows_to = max(1, int(pad_rows_to))
        self._record_stream = None
        self._graph_generation = (-1, -1)
        self.graph_replays = 0
        self.graphs_recorded = 0

    # ---- construction -----------------------------------------------------
    @classmethod
    def from_dir(cls, model_dir, strict_weights: bool = False, **kw) -> "Engine":
        """Model class, sizes and constants come from config.json; weights from
        the folder's safetensors files.  Stored tensors that the model does not
        use are reported in one line, or refused when `strict_weights`."""
        arch, cfg, spec = load_config(model_dir)
        eng = cls(spec, config=cfg, **kw)
        eng.unused_weights = load_into(eng.model, model_dir, aliases=arch.weight_aliases, strict=strict_weights)
        eng._make_cache()
        return eng

    @classmethod
    def from_random(cls, config: Dict[str, Any], seed: int, **kw) -> "Engine":
        """Random weights drawn straight on the device (no files): for
        measurements at sizes where writing a checkpoint first would only cost time.
        The numbers differ from those that `weights.write_random_model` writes for the
        same seed: the device's and the host's random generators are two different ones."""
        arch = lookup(architecture_name(config))
        cfg = arch.config_from_dict(config)
        spec = arch.model_spec(cfg)
        eng = cls(spec, config=cfg, **kw)
        expected = eng.model.expected_params()
        stored = torch.float32 if eng.rt.dtype is torch.float32 else torch.bfloat16

        def get(name):
            return random_tensor(seed, name, expected[name], stored, device=eng.rt.device)

        eng.model.load_params(get)
        eng._make_cache()
        return eng

    def _group_page_bytes(self) -> List[int]:
        """Bytes that one page takes in every entry of each page group."""
        needs, sources = self.model.cache_needs()
        groups = group_needs(needs, sources)
        from ..parts.base import needs_of
        out = [0] * len(groups)
        for n, s in zip(needs, sources):
            paged = needs_of(n)[0] if s is None and n is not None else None
            if paged is not None:
                out[groups.index(paged)] += paged.bytes_per_token(self.rt.dtype) * self.page_size
        return out

    def _make_cache(self) -> None:
        """The pools' sizes.  Given `num_pages` (a number for every group, or one per group),
        `max_tokens` or LLAISYS_NUM_BLOCKS, every group gets that many pages.  Otherwise the memory
        that is free decides: a windowed group gets what `max_seqs` requests can hold at a time,
        ceil(window / page) + 2 pages each, plus the pages of `step_tokens` new tokens (a step's
        portions are held whole until the step is over); the groups that keep all keys share the rest,
        up to `max_seqs` requests of the model's full length."""
        needs, sources = self.model.cache_needs()
        groups = group_needs(needs, sources)
        pages = self._num_pages
        env_pages = os.environ.get("LLAISYS_NUM_BLOCKS", "").strip()
        if pages is None and self._max_tokens is None and env_pages:
            # the reference's switch for its pool size (src/llaisys/models/qwen2.cpp:121)
            if not env_pages.isdigit() or int(env_pages) <= 0:
                raise ValueError(f"LLAISYS_NUM_BLOCKS must be a positive number of pages, found {env_pages!r}")
            pages = int(env_pages)
        if pages is None and self._max_tokens is not None:
            pages = -(-int(self._max_tokens) // self.page_size)
        if pages is None:
            P = self.page_size
            per_seq = -(-self.spec.max_positions // P)
            full = per_seq * self.max_seqs
            pages = [full if g.window <= 0 else
                     min(full, self.max_seqs * (-(-g.window // P) + 2) + -(-self.step_tokens // P)) for g in groups]
            if self.rt.device.type == "cuda" and groups:
                free, _ = torch.cuda.mem_get_info(self.rt.device)
                bpp = [max(1, b) for b in self._group_page_bytes()]
                budget = int(free * 0.85)
                windowed = sum(n * b for n, b, g in zip(pages, bpp, groups) if g.window > 0)
                if windowed > budget // 2:                # (windows as long as the contexts: no group is small)
                    share = max(1, budget // sum(bpp))
                    pages = [min(n, share) for n in pages]
                else:
                    rest = sum(b for b, g in zip(bpp, groups) if g.window <= 0)
                    share = max(1, (budget - windowed) // max(1, rest))
                    pages = [n if g.window > 0 else min(n, share) for n, g in zip(pages, groups)]
        self.cache = CacheManager(needs, sources, page_size=self.page_size, num_pages=pages,
                                  max_seqs=self.max_seqs, dtype=self.rt.dtype, device=self.rt.device,
                                  page_order_seed=self._page_order_seed)

    @property
    def row_tile(self) -> int:
        """Rows that the model's kernels take at a time, as its parts report it: what a scheduler
        rounds a step's tokens to."""
        return self.model.batch_needs().row_tile

    # ---- the step ---------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]):
        """Checks the batch; returns (handles, token counts) of the entries, a handle of -1
        standing for a request that is not live yet.  Nothing is changed."""
        if not entries:
            raise StepError("step: empty batch")
        vocab = self.spec.vocab_size
        if len({e.rid for e in entries}) != len(entries):
            seen = set()
            for e in entries:
                if e.rid in seen:
                    raise StepError(f"step: request {e.rid!r} appears twice in one batch")
                seen.add(e.rid)
        counts = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=len(entries))
        for e, n in zip(entries, counts):
            if n == 1:                               # a decoded token: the common case, checked without arrays
                t = e.tokens[0]
                ok = isinstance(t, (int, np.integer)) and not isinstance(t, bool) and 0 <= t < vocab
                if e.take is not None:
                    k = e.take[0] if len(e.take) == 1 else None
                    if not (isinstance(k, (int, np.integer)) and not isinstance(k, bool) and -1 <= k < FEEDBACK_SLOTS):
                        raise StepError(f"step: request {e.rid!r}: `take` must give, for each of its 1 "
                                        f"tokens, -1 or a place below {FEEDBACK_SLOTS} in the feedback buffer")
                if not ok:
                    raise StepError(f"step: request {e.rid!r} brings a token id outside the vocabulary "
                                    f"of {vocab} (embedding: index out of range)")
                if e.want and (len(e.want) != 1 or int(e.want[0]) != 0):
                    raise StepError(f"step: request {e.rid!r} wants logits at places {list(e.want)} of 1 token")
                continue
            if n == 0:
                raise StepError(f"step: request {e.rid!r} brings no tokens")
            toks = np.asarray(e.tokens)
            if toks.ndim != 1 or toks.dtype.kind not in "iu" or toks.min() < 0 or toks.max() >= vocab:
                raise StepError(f"step: request {e.rid!r} brings a token id outside the vocabulary "
                                f"of {vocab} (embedding: index out of range)")
            if e.take is not None:
                take = np.asarray(e.take)
                if take.shape != (n,) or take.dtype.kind not in "iu" or take.min() < -1 or take.max() >= FEEDBACK_SLOTS:
                    raise StepError(f"step: request {e.rid!r}: `take` must give, for each of its {n} "
                                    f"tokens, -1 or a place below {FEEDBACK_SLOTS} in the feedback buffer")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"step: request {e.rid!r} wants logits at place {w} of {n} tokens")
        handles = self.cache.handles_of([e.rid for e in entries])
        reach = self.cache.cached_many(handles) + counts
        if int(reach.max()) > self.spec.max_positions:
            i = int(np.argmax(reach))
            raise StepError(f"step: request {entries[i].rid!r} would reach {int(reach[i])} positions, the "
                            f"model max sequence length is {self.spec.max_positions}")
        return handles, counts

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits [wanted, vocab] in the order of
        the entries and of their `want` lists, or None when nothing is wanted.
        The tensor may be the output buffer of a recorded step: it is valid until
        the next step (copy it to keep it).
        Raises StepError for a bad batch and CacheFull when pages or slots do
        not suffice; in both cases the cache is as before.  If the model's
        forward itself raises (a size that a kernel refuses), no cached length
        moves, requests that this step admitted are released again, and pages
        reserved for requests that were live already stay with them: the next
        step uses them, or they go back when the request ends."""
        handles, counts = self._validate(entries)
        cache = self.cache
        admitted = []
        try:
            if (handles < 0).any():
                for i, e in enumerate(entries):
                    if handles[i] < 0:
                        cache.admit(e.rid)
                        admitted.append(e.rid)
                        handles[i] = cache.handle(e.rid)
            cache.reserve_many(handles, counts)      # all-or-nothing over the batch
        except CacheFull:
            for rid in admitted:
                cache.release(rid)
            raise
        decode_only = int(counts.max()) == 1
        key = self._graph_key(entries, handles) if decode_only else None
        rows = None
        if key is not None:
            # A recorded step serves one number of requests.  Where requests come and go that number
            # changes every few steps, and most steps would run eagerly or be recorded anew; so a batch
            # is filled up to the next multiple of `pad_rows_to` with copies of its LAST entry: the
            # copies read the same token, position, pages and table row, write the same key and value
            # to the same place, and their logits are dropped.  Not where a mixer keeps state of fixed
            # size (a copy would step the state a second time).
            n = len(entries)
            fill = -n % self.pad_rows_to if (n > self.pad_rows_to and not self.cache.has_state) else 0
            if fill:
                rows = sum(len(e.want) for e in entries)
                last = entries[-1]
                entries = list(entries) + [StepEntry(last.rid, last.tokens, [0], take=last.take)] * fill
                step_handles = np.concatenate([handles, np.full(fill, handles[-1], dtype=handles.dtype)])
                key = (n + fill, key[1] + fill, key[2])
            else:
                step_handles = handles
        if profiler.enabled:
            profiler.phase = "decode" if decode_only else "prefill"
        if self._trace:
            print(f"[litinfer_amd trace] step {self.steps_run}: {len(entries)} requests, "
                  f"{int(counts.sum())} tokens, {sum(len(e.want) for e in entries)} rows of logits, "
                  f"{'recorded' if key is not None else 'eager'}, free pages {cache.free_pages()}",
                  file=sys.stderr, flush=True)
        try:
            if key is None:
                logits = self.model.forward(self._build_context(entries, handles=handles), cache)
            else:
                logits = self._forward_graphed(key, self._build_context(entries, pad_blocks=key[2], handles=step_handles))
                if rows is not None:
                    logits = logits[:rows] if rows else None
        except BaseException:
            for rid in admitted:
                cache.release(rid)
            raise
        cache.commit_many(handles, counts)
        self.steps_run += 1
        return logits

    def finish(self, rid: Hashable) -> None:
        """The request is over: what it holds is given back."""
        if self.cache.has(rid):
            self.cache.release(rid)

    def _build_context(self, entries: Sequence[StepEntry], pad_blocks=None, handles=None) -> StepContext:
        return build_context(self.cache, entries, self.ws, self._uploader, pad_blocks, self.feedback,
                             needs=self.model.batch_needs(), handles=handles)

    # ---- recorded decode steps ----------------------------------------------
    def _graph_key(self, entries: Sequence[StepEntry], handles):
        """(segments, wanted rows, table width per group) of a batch of single tokens
        that may be replayed from a graph, else None.  Table widths are rounded up
        to powers of two so that a graph serves a range of context lengths."""
        if not self.use_graphs or not self.model.graph_safe:
            return None
        widths = tuple(max(16, 1 << (max(need, 1) - 1).bit_length()) for need in self.cache.max_table_len(handles))
        return (len(entries), sum(len(e.want) for e in entries), widths)

    def _record(self, ctx: StepContext):
        """The model's forward pass for `ctx` as a graph (nothing runs).  Recorded on a stream of its own,
        as a capture must be, that waits for the step's stream and is waited for by it; without the
        device-wide wait and the emptying of the allocator's cache that `torch.cuda.graph` begins with:
        where requests come and go a shape is recorded every few steps, the device should not run dry
        for it, and memory handed back to the driver is asked for again a step later."""
        if self._record_stream is None:
            self._record_stream = torch.cuda.Stream(self.rt.device)
        here = torch.cuda.current_stream(self.rt.device)
        self._record_stream.wait_stream(here)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(self._record_stream):
            graph.capture_begin()
            try:
                out = self.model.forward(ctx, self.cache)
            finally:
                graph.capture_end()
        here.wait_stream(self._record_stream)
        return graph, out

    def _buffers_at(self):
        """Changes whenever a buffer that a recorded step may address has moved."""
        return (self.ws.generation, self._uploader.generation)

    def _drop_graphs(self) -> None:
        """Recorded addresses are stale: every shape is recorded anew at its next step (which
        runs eagerly first); how often a shape was seen is kept."""
        for k, state in list(self._graphs.items()):
            if state[0] == "graph":
                self._graphs[k] = ("seen", self.graph_after - 1)

    def _forward_graphed(self, key, ctx: StepContext):
        if self._graph_generation != self._buffers_at():
            self._drop_graphs()                   # a buffer moved since the last decode step
            self._graph_generation = self._buffers_at()
        graphs = self._graphs
        state = graphs.get(key)
        if state is not None and state[0] == "graph":
            graphs.move_to_end(key)
            state[1].replay()
            self.graph_replays += 1
            return state[2]
        # the first steps of a shape run eagerly (the first sizes the buffers); at its graph_after-th the
        # step is recorded and the recording run in the eager pass's place
        seen = 1 if state is None else state[1] + 1
        graphs[key] = ("seen", seen)
        graphs.move_to_end(key)
        logits = None
        if seen >= self.graph_after:
            made = self.ws.allocations
            graph, out = self._record(ctx)
            if self._graph_generation != self._buffers_at() or self.ws.allocations != made:
                # recording itself allocated (the buffer would live in the graph's own pool) or
                # moved a buffer: do not keep it, and nothing recorded before it either
                self._drop_graphs()
                self._graph_generation = self._buffers_at()
                ctx.forget_shared()               # (what the recording prepared has not run)
            else:
                graphs[key] = ("graph", graph, out)
                self.graphs_recorded += 1
                graph.replay()
                logits = out
        if logits is None:
            logits = self.model.forward(ctx, self.cache)
            if self._graph_generation != self._buffers_at():
                # this pass itself made a buffer grow (a larger batch than any before): what was
                # recorded for OTHER shapes addresses the old one
                self._drop_graphs()
                self._graph_generation = self._buffers_at()
        # the least recently used shapes go: a long-lived engine sees hundreds of them, and every
        # recorded one holds its graph and its output buffer
        recorded = sum(1 for s in graphs.values() if s[0] == "graph")
        for k in list(graphs):
            if recorded <= self.max_graphs and len(graphs) <= 8 * self.max_graphs:
                break
            if k != key:
                recorded -= graphs.pop(k)[0] == "graph"
        return logits
