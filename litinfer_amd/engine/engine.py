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
from pathlib import Path
from typing import Any, Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheFull, CacheManager
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
                 config: Any = None, use_graphs: bool = True, graph_after: int = 4,
                 keep_stored_precision: bool = False):
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
        # occurrence and replayed from then on; before that it runs eagerly.  Recording costs about as much
        # as a few steps and drains the queue of work once: where requests come and go and a shape lasts
        # a few steps, recording every shape at its second step costs more than replays give back.
        self.graph_after = max(2, int(graph_after))
        self._trace = trace_enabled()
        self._graphs: Dict[Any, Any] = {}
        self._graph_generation = (-1, -1)
        self.graph_replays = 0

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

    def _bytes_per_page(self) -> int:
        needs, sources = self.model.cache_needs()
        from ..parts.base import PagedNeed
        return sum(n.bytes_per_token(self.rt.dtype) * self.page_size
                   for n, s in zip(needs, sources) if s is None and isinstance(n, PagedNeed))

    def _make_cache(self) -> None:
        needs, sources = self.model.cache_needs()
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
            per_seq = -(-self.spec.max_positions // self.page_size)
            pages = per_seq * self.max_seqs
            if self.rt.device.type == "cuda":
                free, _ = torch.cuda.mem_get_info(self.rt.device)
                bpp = max(1, self._bytes_per_page())
                pages = max(1, min(pages, int(free * 0.85) // bpp))
        self.cache = CacheManager(needs, sources, page_size=self.page_size, num_pages=int(pages),
                                  max_seqs=self.max_seqs, dtype=self.rt.dtype, device=self.rt.device,
                                  page_order_seed=self._page_order_seed)

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
                logits = self._forward_graphed(key, self._build_context(entries, pad_blocks=key[2], handles=handles))
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

    def _forward_graphed(self, key, ctx: StepContext):
        gen = (self.ws.generation, self._uploader.generation)
        state = self._graphs.get(key)
        if state is None or state[0] != "graph" or self._graph_generation != gen:
            if self._graph_generation != gen:
                self._graphs.clear()              # a buffer moved: recorded addresses are stale
                state = None
            # the first steps of a shape run eagerly (the first sizes the buffers), the graph_after-th is recorded
            logits = self.model.forward(ctx, self.cache)
            gen = (self.ws.generation, self._uploader.generation)
            self._graph_generation = gen
            seen = 1 if state is None or state[0] != "seen" else state[1] + 1
            if seen < self.graph_after:
                self._graphs[key] = ("seen", seen)
                return logits
            torch.cuda.synchronize(self.rt.device)
            ctx.forget_shared()                   # what the eager pass prepared must be prepared in the graph too
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out = self.model.forward(ctx, self.cache)
            if (self.ws.generation, self._uploader.generation) != gen:
                self._graphs.clear()              # recording itself moved a buffer: do not keep it
                self._graph_generation = (self.ws.generation, self._uploader.generation)
                return logits
            self._graphs[key] = ("graph", graph, out)
            return logits
        _, graph, out = state
        graph.replay()
        self.graph_replays += 1
        return out
